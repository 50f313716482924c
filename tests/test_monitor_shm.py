"""The lane-idleness table as a cross-process service: the fuselink-monitor daemon owns it in POSIX
shared memory under the reference's layout and names (FuseLink src/monitor.h:23-24, 47-55), this
library attaches as a client, and the REFERENCE's own compiled MonitorClient (oracle/_ref, built from
src/monitor.h where it lies) reads and writes the same table."""
import ctypes as C
import os
import signal
import subprocess
import time

import pytest

from fuselink_amd import build as B
from fuselink_amd import plugin as P

from tests import oracle_binding as ob

IDLE, BUSY, BORROWED = 0, 1, 2


def _lib():
    p = P.NetPlugin(8)
    p.lib.fl_monitor_detach()
    p.lib.fl_monitor_set_clock(0, 0)
    return p


def _status(lib, is_tx, n=16):
    out = (C.c_int32 * n)()
    assert lib.fl_monitor_status(is_tx, n, out) == 0
    return list(out)


def _credits(lib, n, own, idle_credit=4):
    out = (C.c_uint32 * n)()
    assert lib.fl_monitor_credits(n, own, idle_credit, out) == 0
    return list(out)


def _start_daemon(*args):
    exe = B.monitor_path()
    if not os.path.exists(exe):
        pytest.skip("fuselink-monitor is not built")
    proc = subprocess.Popen([exe, "--seconds", "60", *args], stdout=subprocess.PIPE, text=True)
    line = proc.stdout.readline()
    assert "table up" in line, line
    return proc


def _stop(proc):
    proc.send_signal(signal.SIGTERM)
    assert proc.wait(timeout=10) == 0


def _ref_client():
    path = os.path.join(ob.ORACLE_DIR, "_ref", "libref_monitor.so")
    if not os.path.exists(path):
        pytest.skip("oracle/_ref/libref_monitor.so not built (the reference tree is not present)")
    return C.CDLL(path)


def test_attach_without_daemon_fails_loudly():
    p = _lib()
    name = f"/fl_absent_{os.getpid()}".encode()
    rc = p.lib.fl_monitor_attach_shm(name, name, 0)
    assert rc == -6  # FLH_E_STATE
    assert p.lib.fl_monitor_is_shared() == 0


def test_daemon_ages_lanes_and_client_sees_it():
    shm, sem = f"/fl_shm_{os.getpid()}".encode(), f"/fl_sem_{os.getpid()}".encode()
    proc = _start_daemon("--shm", shm.decode(), "--sem", sem.decode())
    p = _lib()
    try:
        assert p.lib.fl_monitor_attach_shm(shm, sem, 0) == 0
        assert p.lib.fl_monitor_is_shared() == 1 and p.lib.fl_monitor_daemon_running() == 1
        now = p.lib.fl_monitor_now()
        # a stamp in the future keeps the lane BUSY through the daemon's ticks; a current one is aged
        assert p.lib.fl_monitor_mark_active(3, 1, now + 30_000_000) == 0
        assert p.lib.fl_monitor_mark_active(5, 1, now) == 0
        assert p.lib.fl_monitor_mark_active(6, 0, now) == 0
        time.sleep(0.05)  # >> MONITOR_TIMEOUT_US = 160 us
        tx, rx = _status(p.lib, 1), _status(p.lib, 0)
        assert tx[3] == BUSY and tx[5] == IDLE and rx[6] == IDLE
        assert _credits(p.lib, 8, own=0) == [4, 4, 4, 0, 4, 4, 4, 4]
        assert _credits(p.lib, 8, own=3) == [4, 4, 4, 1, 4, 4, 4, 4]  # the own lane never drops to 0
        # a BORROWED lane whose stamp is old goes back to IDLE as well (src/monitor.cpp:171-186)
        assert p.lib.fl_monitor_set_entry(9, 1, BORROWED, now) == 0
        time.sleep(0.05)
        assert _status(p.lib, 1)[9] == IDLE
    finally:
        p.lib.fl_monitor_detach()
        _stop(proc)
    # the daemon removed its objects on the way out
    assert p.lib.fl_monitor_attach_shm(shm, sem, 0) == -6


def test_reference_client_and_library_share_one_table():
    """No daemon: this process owns the table (create = 1) and never ticks, so every transition seen
    is one that the other side made."""
    ref = _ref_client()
    p = _lib()
    assert p.lib.fl_monitor_attach_shm(None, None, 1) == 0
    try:
        assert ref.ref_mon_attach() == 0
        out = (C.c_int * 16)()
        # reference marks -> library reads
        ref.ref_mon_mark_tx(2, 0)
        ref.ref_mon_mark_rx(11, 0)
        assert _status(p.lib, 1) == [BUSY if i == 2 else IDLE for i in range(16)]
        assert _status(p.lib, 0) == [BUSY if i == 11 else IDLE for i in range(16)]
        assert _credits(p.lib, 8, own=0) == [4, 4, 0, 4, 4, 4, 4, 4]
        # library marks -> reference reads
        assert p.lib.fl_monitor_mark_active(7, 1, p.lib.fl_monitor_now()) == 0
        ref.ref_mon_status(16, out)
        assert list(out) == [BUSY if i in (2, 7) else IDLE for i in range(16)]
        # the reference's borrow scan (all idle lanes outside the group, last one returned) and the
        # library's restatement of it act on the same table and agree
        assert ref.ref_mon_idle_pick_tx(0, 0) == 15
        assert _status(p.lib, 1) == [IDLE] + [BUSY if i in (2, 7) else BORROWED for i in range(1, 16)]
        assert p.lib.fl_monitor_idle_pick(1, 0, 0, 0) == -1  # nothing left to borrow
        assert p.lib.fl_monitor_idle_pick(0, 11, 0x00F0, 1) == 4  # rx side, masked, first fit
        # library's tick (the daemon's loop body) -> reference sees IDLE everywhere
        assert p.lib.fl_monitor_tick(p.lib.fl_monitor_now() + 1_000_000) == 0
        ref.ref_mon_status(16, out)
        assert list(out) == [IDLE] * 16
    finally:
        ref.ref_mon_detach()
        p.lib.fl_monitor_detach()


def test_reference_client_against_the_daemon():
    ref = _ref_client()
    proc = _start_daemon()
    try:
        assert ref.ref_mon_attach() == 0
        out = (C.c_int * 16)()
        ref.ref_mon_mark_tx(4, 0)  # stamped with the reference's own clock: aged after 160 us
        time.sleep(0.05)
        ref.ref_mon_status(16, out)
        assert list(out) == [IDLE] * 16
        # borrowed lanes stay BORROWED until their (zero) stamp is seen as old: at once
        assert ref.ref_mon_idle_pick_tx(3, 0) == 15
        time.sleep(0.05)
        ref.ref_mon_status(16, out)
        assert list(out) == [IDLE] * 16
    finally:
        ref.ref_mon_detach()
        _stop(proc)


def test_plugin_reads_credits_from_the_daemon():
    p = _lib()
    # without a daemon the plugin refuses to start rather than run on a private table
    os.environ["NCCL_FUSELINK_MONITOR_SHM"] = "1"
    try:
        assert p.lib.fl_net_reset() == 0
        assert p.init() == P.ncclSystemError
        proc = _start_daemon()
        try:
            assert p.init() == P.ncclSuccess
            assert p.lib.fl_monitor_is_shared() == 1
            # a lane that another process keeps busy gets no chunks of the next transfer
            far = p.lib.fl_monitor_now() + 30_000_000
            p.lib.fl_monitor_mark_active(2, 1, far)
            time.sleep(0.01)
            assert _credits(p.lib, 8, own=0) == [4, 4, 0, 4, 4, 4, 4, 4]
        finally:
            assert p.lib.fl_net_reset() == 0  # detaches
            assert p.lib.fl_monitor_is_shared() == 0
            _stop(proc)
    finally:
        os.environ.pop("NCCL_FUSELINK_MONITOR_SHM", None)
        p.lib.fl_net_reset()
        assert p.init() == P.ncclSuccess


def test_a_semaphore_nobody_releases_does_not_stall_the_library():
    """A process that dies while it holds the named semaphore leaves it at zero for ever; the reference's
    sem_wait (src/monitor.h:195) then blocks every client.  Here the wait is bounded and the access goes ahead."""
    shm, sem = f"/fl_shm_dead_{os.getpid()}".encode(), f"/fl_sem_dead_{os.getpid()}".encode()
    p = _lib()
    try:
        assert p.lib.fl_monitor_attach_shm(shm, sem, 1) == 0      # create the table here, as the daemon would
        assert p.lib.fl_monitor_mark_active(2, 1, 123) == 0
        # take the semaphore the way a crashed client would have: wait on it and never post
        libc = C.CDLL(None, use_errno=True)
        libc.sem_open.restype = C.c_void_p
        libc.sem_open.argtypes = [C.c_char_p, C.c_int]
        libc.sem_wait.argtypes = [C.c_void_p]
        libc.sem_post.argtypes = [C.c_void_p]
        h = libc.sem_open(sem, 0)
        assert h and libc.sem_wait(h) == 0
        t0 = time.time()
        assert _status(p.lib, 1)[2] == BUSY                        # answered, after the bounded wait
        waited = time.time() - t0
        assert 0.1 < waited < 5.0, waited
        libc.sem_post(h)
        t0 = time.time()
        assert _status(p.lib, 1)[2] == BUSY
        assert time.time() - t0 < 0.1                              # and at once when the semaphore is free again
    finally:
        p.lib.fl_monitor_detach()
