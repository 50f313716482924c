"""The plugin ABI driven the way NCCL's proxy drives it, with host memory (NCCL_PTR_HOST) so that
the request machinery, the FIFO handshake and the error convention are checked without a GPU.
Host buffers are never staged (FuseLink src/fuselink.cc:8-13), so no kernel is involved here."""
import ctypes as C
import os

import numpy as np
import pytest

from fuselink_amd import plugin as P


@pytest.fixture()
def net():
    p = P.NetPlugin(8)
    assert p.init() == P.ncclSuccess
    p.lib.fl_monitor_reset()
    p.set_credits([])
    return p


def _host(n, seed=0):
    a = np.random.default_rng(seed).integers(0, 256, size=n, dtype=np.uint8)
    return a, a.ctypes.data


def test_library_exports_every_declared_symbol():
    import re, os
    lib = C.CDLL(P.lib_path())
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    names = set()
    for hdr in ("fuselink_hip.h", "fuselink_net.h"):
        text = open(os.path.join(root, "include", hdr)).read()
        names |= set(re.findall(r"\b(flh_[a-z0-9_]+|fl_net_[a-z0-9_]+|fl_monitor_[a-z0-9_]+)\s*\(", text))
        names |= set(re.findall(r"extern\s+\w+\s+(ncclNetPlugin_v\d)\s*;", text))
    assert len(names) > 40
    for n in sorted(names):
        assert hasattr(lib, n), f"{n} is declared in include/ but not exported"


def test_library_shares_no_thread_local_variable_between_its_translation_units():
    """A thread_local variable declared extern in one translation unit and defined in another is reached
    through a wrapper that tests the address of the variable's (absent) initialiser, a weak hidden symbol;
    in a shared object that address is computed relative to the load address, is never null, and gets
    called.  Such state is reached through accessor functions here; the symbol table must show no
    thread-local initialiser or wrapper."""
    import shutil
    import subprocess
    nm = shutil.which("nm")
    if not nm:
        pytest.skip("nm not available")
    out = subprocess.run([nm, P.lib_path()], capture_output=True, text=True, check=True).stdout
    bad = [l for l in out.splitlines() if " _ZTH" in l or " _ZTW" in l]
    assert not bad, bad


@pytest.mark.parametrize("version", [6, 7, 8])
def test_tables_and_properties(version):
    p = P.NetPlugin(version)
    assert p.name == "FuseLink"  # src/plugin.cc:1998
    assert p.init() == P.ncclSuccess
    rc, n = p.devices()
    assert rc == P.ncclSuccess and n == 8
    rc, props = p.getProperties(3)
    assert rc == P.ncclSuccess
    assert props.name == b"fuselink3" and props.guid == 3
    assert props.ptrSupport == P.NCCL_PTR_HOST | P.NCCL_PTR_CUDA | P.NCCL_PTR_DMABUF   # src/plugin.cc:364-370
    assert props.maxRecvs == 1 and props.latency == 0
    if version >= 7:
        assert props.netDeviceType == 0 and props.netDeviceVersion == 0  # src/plugin.cc:376-377
        assert not p.t.getDeviceMr and not p.t.irecvConsumed            # src/plugin.cc:2015-2016
    if version == 8:
        assert props.regIsGlobal == 1
    assert p.getProperties(99)[0] == P.ncclInvalidArgument


def test_connect_accept_are_nonblocking_and_staged(net):
    rc, handle, lcomm = net.listen(0)
    assert rc == P.ncclSuccess and lcomm
    rc, r = net.accept(lcomm)
    assert rc == P.ncclSuccess and r is None           # nobody connected yet
    rc, s = net.connect(0, handle)
    assert rc == P.ncclSuccess and s is None           # posted, peer has not accepted
    rc, s = net.connect(0, handle)
    assert rc == P.ncclSuccess and s is None
    rc, r = net.accept(lcomm)
    assert rc == P.ncclSuccess and r
    rc, s = net.connect(0, handle)
    assert rc == P.ncclSuccess and s
    assert net.closeSend(s) == 0 and net.closeRecv(r) == 0 and net.closeListen(lcomm) == 0


def test_connect_learns_that_its_listener_closed(net):
    # a connect that was posted but never accepted: closing the listen comm must not leave the connecting
    # side polling for ever, and the connection's memory is released (reset refuses while a link is alive)
    rc, handle, lcomm = net.listen(0)
    rc, s = net.connect(0, handle)
    assert rc == P.ncclSuccess and s is None
    assert net.closeListen(lcomm) == 0
    rc, s = net.connect(0, handle)
    assert rc == P.ncclSystemError and s is None
    assert net.lib.fl_net_reset() == 0
    assert net.init() == 0


def test_channel_ids_count_up_per_listen(net):
    # ncclIbListen hands out a global, increasing channelId (src/plugin.cc:693-708); it sits in the handle
    ids = []
    comms = []
    for _ in range(3):
        rc, handle, lcomm = net.listen(1)
        ids.append(int.from_bytes(handle.raw[16:20], "little", signed=True))
        comms.append(lcomm)
    assert ids[1] == ids[0] + 1 and ids[2] == ids[0] + 2
    for c in comms:
        net.closeListen(c)


def test_send_recv_roundtrip_and_sizes(net):
    lcomm, s, r = net.connect_pair(0)
    src, sp = _host(1 << 20, 1)
    dst = np.zeros(1 << 20, dtype=np.uint8)
    rc, smh = net.regMr(s, sp, src.size, P.NCCL_PTR_HOST)
    assert rc == 0 and smh
    rc, rmh = net.regMr(r, dst.ctypes.data, dst.size, P.NCCL_PTR_HOST)
    assert rc == 0 and rmh
    # the sender cannot proceed before the receive is posted (src/plugin.cc:1510-1514)
    rc, req = net.isend(s, sp, 4096, 7, smh)
    assert rc == 0 and req is None
    rc, rreq = net.irecv(r, [dst.ctypes.data], [1 << 20], [7], [rmh])
    assert rc == 0 and rreq
    rc, done, _ = net.test(rreq)
    assert rc == 0 and done == 0                        # posted, not matched
    rc, sreq = net.isend(s, sp, 1 << 20, 7, smh)
    assert rc == 0 and sreq
    assert net.wait(sreq) is not None
    assert net.wait(rreq) == 1 << 20                    # byte count of the receive is reported
    np.testing.assert_array_equal(dst, src)
    # a shorter send into a larger posted receive is fine and reports the sent size
    rc, rreq = net.irecv(r, [dst.ctypes.data], [1 << 20], [8], [rmh])
    rc, sreq = net.isend(s, sp + 100, 1000, 8, smh)
    assert rc == 0 and sreq
    net.wait(sreq)
    assert net.wait(rreq) == 1000
    np.testing.assert_array_equal(dst[:1000], src[100:1100])
    st = net.comm_stats(s)
    assert st["n_finished"] == 2 and st["in_flight"] == 0
    assert net.deregMr(s, smh) == 0 and net.deregMr(r, rmh) == 0
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_a_nic_in_use_is_stamped_at_most_once_in_a_tenth_of_the_monitors_timeout(net):
    """updateTxChannelActive (src/fuselink.h:247-252) stamps the NIC's table entry on every send; under the table's lock
    that was the busiest line of a process with eight proxy threads.  The plugin stamps an entry at most once in 16 us
    (FL_NET_MONITOR_TIMEOUT_US / 10): the recorded time of last activity may be that much older than the truth, never
    more.  With the clock in hand: a send at t stamps t; one at t + 10 leaves the stamp alone (the entry ages out 160 us
    after t, not after t + 10); one at t + 200 stamps again."""
    L = net.lib
    IDLE, BUSY = 0, 1
    assert net.reconfigure(NCCL_FUSELINK_LANES=8) is None
    lcomm, s, r = net.connect_pair(3)                     # NIC 3
    src, sp = _host(4096, 3)
    dst = np.zeros(4096, dtype=np.uint8)
    _, smh = net.regMr(s, sp, src.size, P.NCCL_PTR_HOST)
    _, rmh = net.regMr(r, dst.ctypes.data, dst.size, P.NCCL_PTR_HOST)

    def send(tag):
        rc, rreq = net.irecv(r, [dst.ctypes.data], [4096], [tag], [rmh])
        assert rc == 0 and rreq
        rc, sreq = net.isend(s, sp, 4096, tag, smh)
        assert rc == 0 and sreq
        net.wait(sreq), net.wait(rreq)

    def tx_status():
        st = (C.c_int32 * 8)()
        assert L.fl_monitor_status(1, 8, st) == 0
        return st[3]

    t = 1_000_000
    try:
        L.fl_monitor_set_clock(1, t)
        send(0)
        assert tx_status() == BUSY
        L.fl_monitor_set_clock(1, t + 10)
        send(1)                                           # within 16 us of the stamp: not stamped again
        L.fl_monitor_tick(t + 165)
        assert tx_status() == IDLE                        # 165 us after t; a stamp at t + 10 would still be 155 us young
        L.fl_monitor_set_clock(1, t + 200)
        send(2)
        assert tx_status() == BUSY
        L.fl_monitor_tick(t + 355)
        assert tx_status() == BUSY                        # stamped at t + 200: 155 us old
        L.fl_monitor_tick(t + 360)
        assert tx_status() == IDLE
    finally:
        L.fl_monitor_set_clock(0, 0)
        net.deregMr(s, smh), net.deregMr(r, rmh)
        net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)
        net.reconfigure(NCCL_FUSELINK_LANES=None)


def test_error_convention(net):
    lcomm, s, r = net.connect_pair(0)
    src, sp = _host(8192, 2)
    dst = np.zeros(8192, dtype=np.uint8)
    _, smh = net.regMr(s, sp, src.size, P.NCCL_PTR_HOST)
    _, rmh = net.regMr(r, dst.ctypes.data, dst.size, P.NCCL_PTR_HOST)
    # send larger than the posted receive -> ncclInvalidUsage (src/plugin.cc:1555-1562)
    rc, rreq = net.irecv(r, [dst.ctypes.data], [1000], [1], [rmh])
    assert rc == 0 and rreq
    rc, sreq = net.isend(s, sp, 2000, 1, smh)
    assert rc == P.ncclInvalidUsage and sreq is None
    # a send with another tag does not match and would block (src/plugin.cc:1552)
    rc, sreq = net.isend(s, sp, 500, 2, smh)
    assert rc == 0 and sreq is None
    rc, sreq = net.isend(s, sp, 500, 1, smh)
    assert rc == 0 and sreq
    net.wait(sreq), net.wait(rreq)
    # grouped receives are rejected (src/plugin.cc:1448-1451, 1873-1880); more than 8 is an error outright (1683)
    rc, q = net.irecv(r, [dst.ctypes.data] * 2, [10, 10], [1, 1], [rmh, rmh])
    assert rc == P.ncclInternalError and q is None
    rc, q = net.irecv(r, [dst.ctypes.data] * 9, [10] * 9, [1] * 9, [rmh] * 9)
    assert rc == P.ncclInternalError
    # buffers outside their registration
    other = np.zeros(64, dtype=np.uint8)
    rc, q = net.isend(s, other.ctypes.data + (1 << 30), 16, 1, smh)
    assert rc in (0, P.ncclInvalidArgument) and q is None
    # test on a request that already completed
    rc, _, _ = net.test(sreq)
    assert rc == P.ncclInternalError
    # unsupported pointer type
    rc, mh = net.regMr(s, sp, 16, 64)
    assert rc == P.ncclInvalidArgument and mh is None
    net.deregMr(s, smh), net.deregMr(r, rmh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_refresh_cadence_gates_posting(net):
    """Every 8 completions the receiver may change lanes, and only once nothing is outstanding
    (src/plugin.cc:38, 1700-1712): at those points a second irecv has to wait for the first."""
    lcomm, s, r = net.connect_pair(0)
    src, sp = _host(4096, 3)
    dst = np.zeros(4096, dtype=np.uint8)
    _, smh = net.regMr(s, sp, src.size, P.NCCL_PTR_HOST)
    _, rmh = net.regMr(r, dst.ctypes.data, dst.size, P.NCCL_PTR_HOST)
    tag = 0
    refreshed_at = []
    while net.comm_stats(r)["n_finished"] < 40:
        fin = net.comm_stats(r)["n_finished"]
        before = net.comm_stats(r)["refreshes"]
        rc, first = net.irecv(r, [dst.ctypes.data], [64], [tag], [rmh])
        assert rc == 0 and first
        if net.comm_stats(r)["refreshes"] != before:
            refreshed_at.append(fin)
        # with one receive outstanding a second one is held back exactly on a batch boundary
        rc, second = net.irecv(r, [dst.ctypes.data + 64], [64], [tag + 1], [rmh])
        assert rc == 0
        assert (second is None) == (fin % 8 == 0), fin
        for q, t in ((first, tag), (second, tag + 1)):
            if q is None:
                continue
            rc, sreq = net.isend(s, sp, 64, t, smh)
            assert rc == 0 and sreq
            net.wait(sreq), net.wait(q)
        tag += 2
    # refreshes happen on the batch boundaries that an irecv actually met with nothing outstanding
    assert refreshed_at and all(f % 8 == 0 for f in refreshed_at) and refreshed_at[0] == 0
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_request_slots_run_out_at_256(net):
    lcomm, s, r = net.connect_pair(0)
    src, sp = _host(4096, 4)
    dst = np.zeros(4096, dtype=np.uint8)
    _, smh = net.regMr(s, sp, src.size, P.NCCL_PTR_HOST)
    _, rmh = net.regMr(r, dst.ctypes.data, dst.size, P.NCCL_PTR_HOST)
    # get n_finished off the refresh boundary first
    _, rreq = net.irecv(r, [dst.ctypes.data], [8], [0], [rmh])
    _, sreq = net.isend(s, sp, 8, 0, smh)
    net.wait(sreq), net.wait(rreq)
    reqs = []
    for k in range(256):
        rc, q = net.irecv(r, [dst.ctypes.data], [8], [k], [rmh])
        assert rc == 0 and q, k
        reqs.append(q)
    rc, q = net.irecv(r, [dst.ctypes.data], [8], [999], [rmh])
    assert rc == P.ncclInternalError and q is None       # src/plugin.cc:1082-1084
    # requests are slots of a fixed table inside the connection: first free first (src/plugin.cc:1070-1085)
    assert len(set(reqs)) == 256
    stride = reqs[1] - reqs[0]
    assert all(reqs[i + 1] - reqs[i] == stride for i in range(255))
    for k in range(256):
        rc, sq = net.isend(s, sp, 8, k, smh)
        assert rc == 0 and sq
        net.wait(sq), net.wait(reqs[k])
    assert net.comm_stats(r)["n_finished"] == 257
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_injected_wire_fault_surfaces_in_test(net):
    lcomm, s, r = net.connect_pair(0)
    src, sp = _host(4096, 5)
    dst = np.zeros(4096, dtype=np.uint8)
    _, smh = net.regMr(s, sp, src.size, P.NCCL_PTR_HOST)
    _, rmh = net.regMr(r, dst.ctypes.data, dst.size, P.NCCL_PTR_HOST)
    _, rreq = net.irecv(r, [dst.ctypes.data], [64], [0], [rmh])
    _, sreq = net.isend(s, sp, 64, 0, smh)
    assert net.lib.fl_net_inject_fault(rreq) == 0
    net.wait(sreq)
    rc, done, _ = net.test(rreq)
    assert rc == P.ncclRemoteError and done == 0        # src/plugin.cc:1839-1861
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_a_failed_request_is_freed_and_the_connection_goes_on(net):
    """The reference returns from a failed completion with the request still allocated (src/plugin.cc:1839-1861); its
    communicator is dead after that.  Here the connection lives on, so the request must be freed and counted: with the
    default cadence of 8 a receive left in flight would hold every later refresh back for ever.  Fault on request 5 of
    20: its test reports ncclRemoteError once, the 19 others arrive, the refreshes at 8 and 16 happen, and both request
    tables are back to 256 free slots."""
    lcomm, s, r = net.connect_pair(0)
    src, sp = _host(20 * 64, 11)
    dst = np.zeros(20 * 64, dtype=np.uint8)
    _, smh = net.regMr(s, sp, src.size, P.NCCL_PTR_HOST)
    _, rmh = net.regMr(r, dst.ctypes.data, dst.size, P.NCCL_PTR_HOST)
    assert net.free_requests(s) == 256 and net.free_requests(r) == 256
    failed = 0
    for k in range(20):
        rreq = None
        for _ in range(1000):
            rc, rreq = net.irecv(r, [dst.ctypes.data + 64 * k], [64], [k], [rmh])
            assert rc == 0
            if rreq:
                break
        assert rreq, f"receive {k} was never accepted: the refresh gate stayed shut"
        rc, sreq = net.isend(s, sp + 64 * k, 64, k, smh)
        assert rc == 0 and sreq
        if k == 5:
            assert net.lib.fl_net_inject_fault(rreq) == 0
        net.wait(sreq)
        rc, done, _ = net.test(rreq)
        if k == 5:
            assert rc == P.ncclRemoteError and done == 0
            failed += 1
            rc, _, _ = net.test(rreq)
            assert rc == P.ncclInternalError          # the request is no longer in flight
        else:
            assert rc == 0 and done == 1
    assert failed == 1
    st = net.comm_stats(r)
    assert st["n_finished"] == 20 and st["in_flight"] == 0 and st["refreshes"] == 3      # at 0, 8 and 16
    assert net.free_requests(s) == 256 and net.free_requests(r) == 256
    np.testing.assert_array_equal(dst, src)
    net.deregMr(s, smh), net.deregMr(r, rmh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_the_senders_mask_is_refreshed_on_the_references_cadence_and_reaches_the_receiver(net):
    """The sender's lane-availability mask (refreshTxUsage / getTxUsage, src/fuselink.h:261-267, placeholders there) is
    refreshed before every send for which (n_finished + 1) % 8 == 0 (src/plugin.cc:1441-1447), travels as the request's
    immediate data (1463) and is kept by the receiver when the receive completes (1884-1885).  With the clock in hand: a
    lane whose send side is busy drops out of the mask at the next refresh, not before, and comes back at the one after
    its stamp has aged out."""
    from tests import oracle_binding as ob
    O = ob.lib()
    L = net.lib
    assert net.reconfigure(NCCL_FUSELINK_LANES=8) is None
    lcomm, s, r = net.connect_pair(2)                    # the comm's own lane is 2
    src, sp = _host(64, 12)
    dst = np.zeros(64, dtype=np.uint8)
    _, smh = net.regMr(s, sp, 64, P.NCCL_PTR_HOST)
    _, rmh = net.regMr(r, dst.ctypes.data, 64, P.NCCL_PTR_HOST)
    t = 3_000_000
    try:
        L.fl_monitor_set_clock(1, t)
        L.fl_monitor_set_entry(5, 1, 1, t + 2000)        # lane 5's send side: BUSY until t + 2160
        due = 0
        for k in range(40):
            if k == 20:
                L.fl_monitor_set_clock(1, t + 3000)      # ... by now it has aged out
            before = net.mask_stats(s)
            rreq = None
            while not rreq:
                rc, rreq = net.irecv(r, [dst.ctypes.data], [64], [k], [rmh])
                assert rc == 0
            rc, sreq = net.isend(s, sp, 64, k, smh)
            assert rc == 0 and sreq
            after = net.mask_stats(s)
            refreshed = after["refreshes"] - before["refreshes"]
            assert refreshed == O.fl_refresh_tx_due(k), k                 # n_finished == k here: one request at a time
            due += refreshed
            # the placeholder's value until the first refresh, then what the send statuses said at the latest one
            exp = 0xffffffff if k < 7 else (0xffffffdf if k < 23 else 0xffffffff)
            assert after["mask"] == exp, (k, hex(after["mask"]))
            net.wait(sreq), net.wait(rreq)
            assert net.mask_stats(r)["mask"] == exp                        # comm->txAvailable = imm_data
        assert due == 5
    finally:
        L.fl_monitor_set_clock(0, 0)
        L.fl_monitor_reset()
        net.deregMr(s, smh), net.deregMr(r, rmh)
        net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)
        net.reconfigure(NCCL_FUSELINK_LANES=None)


def test_regMrDmaBuf_refuses_a_descriptor_that_is_not_a_dmabuf(net, tmp_path):
    """regMrDmaBuf (src/plugin.cc:1168, 1278-1280) gets a descriptor and an offset with the buffer.  No descriptor (-1) is
    a plain registration; a descriptor that is not a DMA-BUF of device memory holding the range is refused, not ignored."""
    lcomm, s, r = net.connect_pair(0)
    src, sp = _host(4096, 13)
    rc, mh = net.regMrDmaBuf(s, sp, 4096, P.NCCL_PTR_HOST, 0, -1)
    assert rc == 0 and mh
    assert net.deregMr(s, mh) == 0
    f = open(tmp_path / "not_a_dmabuf", "w+b")
    f.truncate(1 << 20)
    rc, mh = net.regMrDmaBuf(s, sp, 4096, P.NCCL_PTR_CUDA, 0, f.fileno())      # an ordinary file
    assert rc == P.ncclInvalidArgument and mh is None
    rc, mh = net.regMrDmaBuf(s, sp, 4096, P.NCCL_PTR_HOST, 0, f.fileno())      # and host memory takes no descriptor at all
    assert rc == P.ncclInvalidArgument and mh is None
    f.close()
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_cuda_pointer_fails_loudly_without_gpu(net):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lcomm, s, r = net.connect_pair(0)
    src, sp = _host(4096, 6)
    rc, mh = net.regMr(s, sp, 4096, P.NCCL_PTR_CUDA)
    assert rc == P.ncclUnhandledCudaError and mh is None  # no CPU fallback for device memory
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


@pytest.mark.parametrize("header", ["fuselink_hip.h", "fuselink_net.h"])
def test_headers_are_plain_c(header, tmp_path):
    """The boundary is a C ABI: both headers must compile as C99 with nothing else included before them."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if not gcc:
        pytest.skip("no C compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "use.c"
    src.write_text(f'#include "{header}"\nint main(void) {{ return 0; }}\n')
    res = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-I" + os.path.join(root, "include"), str(src)],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


# ---- the shared-memory wire: the two ends in different processes (NCCL_FUSELINK_WIRE=shm) ---------------------------
_LISTENER = r"""
import sys, time
import numpy as np
from fuselink_amd import plugin as P
p = P.NetPlugin(8)
assert p.init() == P.ncclSuccess
rc, handle, lcomm = p.listen(0)
assert rc == P.ncclSuccess
sys.stdout.write(handle.raw.hex() + "\n"); sys.stdout.flush()
rcomm = None
for _ in range(20000):
    rc, rcomm = p.accept(lcomm)
    assert rc == P.ncclSuccess
    if rcomm:
        break
    time.sleep(0.001)
assert rcomm, "nobody connected"
# host memory does not travel on this wire: registration works, posting a receive is refused
buf = np.zeros(4096, dtype=np.uint8)
rc, mh = p.regMr(rcomm, buf.ctypes.data, buf.nbytes, P.NCCL_PTR_HOST)
assert rc == P.ncclSuccess
rc, req = p.irecv(rcomm, [buf.ctypes.data], [4096], [7], [mh])
assert rc == P.ncclInvalidUsage and not req, (rc, req)
assert p.deregMr(rcomm, mh) == P.ncclSuccess
sys.stdin.readline()   # the connecting side is done
assert p.closeRecv(rcomm) == P.ncclSuccess
assert p.closeListen(lcomm) == P.ncclSuccess
print("listener ok")
"""


def test_two_processes_meet_through_the_handle_alone():
    """listen in a child process, connect here with nothing but the 128 bytes it printed (NCCL's bootstrap carries
    them between ranks): the staged connect returns no comm until the listener has accepted, as the reference's does
    (FuseLink src/plugin.cc:407-423, 721-760), and the shared-memory object's name is gone once both ends hold it."""
    import subprocess
    import sys
    import time
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, NCCL_FUSELINK_WIRE="shm", PYTHONPATH=root)
    child = subprocess.Popen([sys.executable, "-c", _LISTENER], stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                             text=True, env=env, cwd=root)
    try:
        line = child.stdout.readline().strip()
        assert len(line) == 2 * P.NCCL_NET_HANDLE_MAXSIZE, child.stderr.read()
        handle = C.create_string_buffer(bytes.fromhex(line), P.NCCL_NET_HANDLE_MAXSIZE)
        name = handle.raw[40:104].split(b"\0")[0].decode()
        assert name.startswith("/fuselink-wire-")
        old = os.environ.get("NCCL_FUSELINK_WIRE")
        p = P.NetPlugin(8)
        p.reconfigure(NCCL_FUSELINK_WIRE="shm")
        try:
            scomm = None
            for _ in range(20000):
                rc, scomm = p.connect(1, handle)
                assert rc == P.ncclSuccess
                if scomm:
                    break
                time.sleep(0.001)
            assert scomm, "the listener never accepted"
            assert not os.path.exists("/dev/shm" + name)   # unlinked at accept: nothing is left behind if a process dies
            buf, ptr = _host(4096)
            rc, mh = p.regMr(scomm, ptr, buf.nbytes, P.NCCL_PTR_HOST)
            assert rc == P.ncclSuccess
            rc, req = p.isend(scomm, ptr, 4096, 7, mh)
            assert rc == P.ncclInvalidUsage and not req
            assert p.deregMr(scomm, mh) == P.ncclSuccess
            assert p.closeSend(scomm) == P.ncclSuccess
        finally:
            p.reconfigure(NCCL_FUSELINK_WIRE=old)
        child.stdin.write("done\n")
        child.stdin.flush()
        out, err = child.communicate(timeout=60)
        assert child.returncode == 0 and "listener ok" in out, err
    finally:
        if child.poll() is None:
            child.kill()


def test_a_listener_that_never_accepts_leaves_no_shared_memory_behind():
    p = P.NetPlugin(8)
    old = os.environ.get("NCCL_FUSELINK_WIRE")
    p.reconfigure(NCCL_FUSELINK_WIRE="shm")
    try:
        rc, handle, lcomm = p.listen(0)
        assert rc == P.ncclSuccess
        name = handle.raw[40:104].split(b"\0")[0].decode()
        assert os.path.exists("/dev/shm" + name)
        assert p.lib.fl_net_reset() != 0               # an open listener of this wire holds off a reset too
        assert p.closeListen(lcomm) == P.ncclSuccess
        assert not os.path.exists("/dev/shm" + name)
        assert p.lib.fl_net_reset() == 0 and p.init() == P.ncclSuccess
        # a connect with the stale handle fails cleanly
        rc, scomm = p.connect(0, handle)
        assert rc == P.ncclSystemError and not scomm
    finally:
        p.reconfigure(NCCL_FUSELINK_WIRE=old)


def test_the_shared_memory_wire_refuses_a_listener_in_the_connecting_process():
    p = P.NetPlugin(8)
    old = os.environ.get("NCCL_FUSELINK_WIRE")
    p.reconfigure(NCCL_FUSELINK_WIRE="shm")
    try:
        rc, handle, lcomm = p.listen(0)
        assert rc == P.ncclSuccess
        rc, scomm = p.connect(0, handle)
        assert rc == P.ncclInvalidUsage and not scomm
        rc, rcomm = p.accept(lcomm)
        assert rc == P.ncclSuccess and not rcomm       # nobody connected
        assert p.closeListen(lcomm) == P.ncclSuccess
    finally:
        p.reconfigure(NCCL_FUSELINK_WIRE=old)


def test_the_shared_memory_wire_refuses_an_object_of_another_size():
    """The wire's layout belongs to the build; a listener of another build would lay the object out differently.  A
    connect that finds an object of another size refuses it instead of mapping it."""
    p = P.NetPlugin(8)
    old = os.environ.get("NCCL_FUSELINK_WIRE")
    p.reconfigure(NCCL_FUSELINK_WIRE="shm")
    name = "/fuselink-wire-1-999999"
    path = "/dev/shm" + name
    try:
        rc, handle, lcomm = p.listen(0)
        assert rc == P.ncclSuccess
        with open(path, "wb") as f:
            f.write(b"\0" * 4096)
        forged = C.create_string_buffer(handle.raw, P.NCCL_NET_HANDLE_MAXSIZE)
        forged[40:104] = name.encode().ljust(64, b"\0")
        rc, scomm = p.connect(0, forged)
        assert rc == P.ncclInvalidUsage and not scomm
        assert p.closeListen(lcomm) == P.ncclSuccess
    finally:
        if os.path.exists(path):
            os.unlink(path)
        p.reconfigure(NCCL_FUSELINK_WIRE=old)
