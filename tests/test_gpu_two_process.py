"""Sender and receiver of a connection in different processes (NCCL_FUSELINK_WIRE=shm), driven through the plugin table
from Python on both sides: the receiving process is a child that listens, prints the 128-byte handle, accepts, posts its
receives and compares what arrived with the seeded pattern; this process connects with the handle alone, sends, and
checks the chunk -> lane table that its striping launch wrote against the CPU oracle, request by request, with the
credit epoch's prefix carried from one request to the next."""
import json
import os
import subprocess
import sys
import time

import numpy as np
import pytest

from fuselink_amd import plugin as P
from tests import oracle_binding as ob

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

_RECEIVER = r"""
import json, sys, time
import numpy as np
import torch
from fuselink_amd import plugin as P
sizes, seed = json.loads(sys.argv[1]), int(sys.argv[2])
p = P.NetPlugin(8)
assert p.init() == P.ncclSuccess
rc, handle, lcomm = p.listen(0)
assert rc == P.ncclSuccess
sys.stdout.write(handle.raw.hex() + "\n"); sys.stdout.flush()
rcomm = None
deadline = time.time() + 60
while not rcomm:
    rc, rcomm = p.accept(lcomm)
    assert rc == P.ncclSuccess and time.time() < deadline
total = sum(sizes)
dst = torch.zeros(total + 64, dtype=torch.uint8, device="cuda")
rc, mh = p.regMr(rcomm, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
assert rc == P.ncclSuccess
ahead = len(sys.argv) > 3 and sys.argv[3] == "ahead"   # after the first request, post every receive before testing any
off, posted = 0, []
for q, n in enumerate(sizes):
    req = None
    while not req:                      # (the refresh gate may hold a receive back until the one before it is done)
        rc, req = p.irecv(rcomm, [dst.data_ptr() + off], [n], [q], [mh])
        assert rc == P.ncclSuccess and time.time() < deadline
    posted.append((q, n, req))
    off += n
    if ahead and 0 < q < len(sizes) - 1:
        continue
    for q2, n2, r2 in posted:
        done = 0
        while not done:
            rc, done, got = p.test(r2)
            assert rc == P.ncclSuccess and time.time() < deadline
        assert got == n2, (q2, got, n2)
    posted = []
torch.cuda.synchronize()
exp = np.random.default_rng(seed).integers(1, 256, size=total, dtype=np.uint8)
back = dst.cpu().numpy()
assert np.array_equal(back[:total], exp), "received bytes differ from what was sent"
assert not back[total:].any(), "bytes behind the last request were touched"
print("receiver ok"); sys.stdout.flush()
sys.stdin.readline()                    # the sender has closed its comm
assert p.deregMr(rcomm, mh) == P.ncclSuccess
assert p.closeRecv(rcomm) == P.ncclSuccess and p.closeListen(lcomm) == P.ncclSuccess
"""


def _run_pair(env, sizes, seed, credits, lanes, chunk, window_bytes):
    import torch
    env = dict(os.environ, NCCL_FUSELINK_WIRE="shm", PYTHONPATH=ROOT, **{k: str(v) for k, v in env.items()})
    child = subprocess.Popen([sys.executable, "-c", _RECEIVER, json.dumps(sizes), str(seed)], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                             stderr=subprocess.PIPE, text=True, env=env, cwd=ROOT)
    keys = ["NCCL_FUSELINK_WIRE"] + list(env_keys(env))
    p = P.NetPlugin(8)
    try:
        line = child.stdout.readline().strip()
        assert len(line) == 2 * P.NCCL_NET_HANDLE_MAXSIZE, child.stderr.read()[-3000:]
        import ctypes as C
        handle = C.create_string_buffer(bytes.fromhex(line), P.NCCL_NET_HANDLE_MAXSIZE)
        p.reconfigure(**{k: env[k] for k in keys})
        scomm, deadline = None, time.time() + 60
        while not scomm:
            rc, scomm = p.connect(1, handle)
            assert rc == P.ncclSuccess and time.time() < deadline
        total = sum(sizes)
        src_np = np.random.default_rng(seed).integers(1, 256, size=total, dtype=np.uint8)
        src = torch.from_numpy(src_np).cuda()
        rc, mh = p.regMr(scomm, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
        assert rc == P.ncclSuccess
        off, epoch, chunks_before = 0, 0, 0
        for q, n in enumerate(sizes):
            req = None
            while not req:                  # no request while the receive has not been posted
                rc, req = p.isend(scomm, src.data_ptr() + off, n, q, mh)
                assert rc == P.ncclSuccess and time.time() < deadline
            done = 0
            while not done:
                rc, done, _ = p.test(req)
                assert rc == P.ncclSuccess and time.time() < deadline
            # the table of the request's last wave: what the oracle schedules for those chunks from the carried state
            rows, hdr = p.last_table(scomm)
            exp_all, _, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=n, chunk_bytes=chunk,
                                               mode=ob.SCHED_RESET_OFFSETS, state=_state(epoch, chunks_before))
            waves = _waves(exp_all, lanes, window_bytes, chunk)
            first = waves[-1]
            exp, _, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=n - int(exp_all["src_off"][first]),
                                           chunk_bytes=chunk, src_base=int(exp_all["src_off"][first]), mode=ob.SCHED_RESET_OFFSETS,
                                           state=_state(epoch + int(exp_all["src_off"][first]), chunks_before + first))
            assert rows.size == exp.size, (q, rows.size, exp.size)
            for f in ("src_off", "win_off", "len", "lane"):
                np.testing.assert_array_equal(rows[f], exp[f], err_msg=f"request {q}, {f}")
            off += n
            epoch += n
            chunks_before += (n + chunk - 1) // chunk
        assert child.stdout.readline().strip() == "receiver ok", child.stderr.read()[-3000:]
        assert p.deregMr(scomm, mh) == P.ncclSuccess and p.closeSend(scomm) == P.ncclSuccess
        child.stdin.write("closed\n")
        child.stdin.flush()
        _, err = child.communicate(timeout=60)
        assert child.returncode == 0, err[-3000:]
    finally:
        if child.poll() is None:
            child.kill()
        p.reconfigure(**{k: None for k in keys})


def env_keys(env):
    return [k for k in env if k.startswith("NCCL_FUSELINK_") and k not in ("NCCL_FUSELINK_WIRE", "NCCL_FUSELINK_TEST_HOOKS")]


def _state(epoch_bytes, chunk_index):
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["epoch_bytes"] = epoch_bytes
    st["chunk_index"] = chunk_index
    return st


def _waves(table, lanes, window_bytes, chunk):
    """First chunk of every wave of a request: a wave takes as many of the remaining chunks as leave no lane with more
    chunks than its window holds (the plugin's rule, from the credit row's closed form; here counted off the oracle's
    table), 4096 at most."""
    per_lane = window_bytes // chunk
    starts, i, n = [], 0, len(table)
    while i < n:
        starts.append(i)
        count = np.zeros(lanes, dtype=np.int64)
        j = i
        while j < n and j - i < 4096 and count[int(table["lane"][j])] < per_lane:
            count[int(table["lane"][j])] += 1
            j += 1
        assert j > i
        i = j
    return starts


DIRECT = pytest.mark.parametrize("direct", [1, 0])   # written into the posted buffers through their registrations / through the landing windows


@DIRECT
def test_cfg1_shape_tables_and_bytes_across_two_processes(direct):
    # the reference's experiment: 4 MiB in 512 KiB chunks over 2 lanes; then requests that start mid-round and a ragged one
    chunk = 512 << 10
    _run_pair({"NCCL_FUSELINK_LANES": 2, "NCCL_FUSELINK_CHUNKSIZE": chunk, "NCCL_FUSELINK_CREDITS": "1,1", "NCCL_FUSELINK_REFRESH_BATCH": 1000, "NCCL_FUSELINK_WIRE_DIRECT": direct},
              [4 << 20, 5 * chunk, 3 * chunk + 777, chunk], seed=31, credits=[1, 1], lanes=2, chunk=chunk, window_bytes=8 << 20)


@DIRECT
def test_cfg2_shape_tables_and_bytes_across_two_processes(direct):
    # 64 MiB in 256 KiB chunks over 8 lanes with uneven credits; windows of 56 MiB per lane hold the message in one wave
    chunk = 256 << 10
    credits = [8, 6, 7, 1, 8, 7, 3, 3]
    _run_pair({"NCCL_FUSELINK_LANES": 8, "NCCL_FUSELINK_CHUNKSIZE": chunk, "NCCL_FUSELINK_CREDITS": ",".join(map(str, credits)),
               "NCCL_FUSELINK_WINDOW_UNITS": 28, "NCCL_FUSELINK_REFRESH_BATCH": 1000, "NCCL_FUSELINK_WIRE_DIRECT": direct},
              [64 << 20, 9 * chunk + 5], seed=32, credits=credits, lanes=8, chunk=chunk, window_bytes=56 << 20)


@DIRECT
def test_waves_through_small_windows_across_two_processes(direct):
    # 2 MiB windows per lane, three sets of landing windows: requests of several waves, the table is the last wave's
    chunk = 128 << 10
    credits = [3, 1, 2, 2]
    _run_pair({"NCCL_FUSELINK_LANES": 4, "NCCL_FUSELINK_CHUNKSIZE": chunk, "NCCL_FUSELINK_CREDITS": ",".join(map(str, credits)),
               "NCCL_FUSELINK_WINDOW_UNITS": 1, "NCCL_FUSELINK_WIRE_SETS": 3, "NCCL_FUSELINK_REFRESH_BATCH": 1000, "NCCL_FUSELINK_WIRE_DIRECT": direct},
              [20 << 20, (7 << 20) + 4321, 3 * chunk], seed=33, credits=credits, lanes=4, chunk=chunk, window_bytes=2 << 20)


@DIRECT
def test_requests_that_wait_together_share_a_wave_across_two_processes(direct):
    """NCCL keeps eight 512 KiB steps in flight; a wave per request would cost both processes their launches and events
    for half a megabyte each.  Requests that wait together, of whole chunks and under one credit row, travel as one wave:
    staged by one launch as one message from the carried prefix on, carried by one, reassembled by one.  The receiver
    posts four receives before it tests any, the sender matches all four before its first test; the table its striping
    launch wrote must be the oracle's schedule of the 2.5 MiB the four requests make up, the bytes must arrive."""
    import ctypes as C
    import torch
    lanes, chunk = 4, 128 << 10
    credits = [3, 1, 2, 2]
    sizes = [3 * chunk, 4 * chunk, 2 * chunk, 8 * chunk, 3 * chunk + 999, chunk]      # first on its own, four together (the last of them ragged), one behind
    env = dict(os.environ, NCCL_FUSELINK_WIRE="shm", PYTHONPATH=ROOT, NCCL_FUSELINK_LANES=str(lanes), NCCL_FUSELINK_CHUNKSIZE=str(chunk),
               NCCL_FUSELINK_CREDITS=",".join(map(str, credits)), NCCL_FUSELINK_REFRESH_BATCH="1000", NCCL_FUSELINK_WIRE_DIRECT=str(direct))
    child = subprocess.Popen([sys.executable, "-c", _RECEIVER, json.dumps(sizes), "34", "ahead"], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                             stderr=subprocess.PIPE, text=True, env=env, cwd=ROOT)
    keys = ["NCCL_FUSELINK_WIRE"] + list(env_keys(env))
    p = P.NetPlugin(8)
    try:
        line = child.stdout.readline().strip()
        assert len(line) == 2 * P.NCCL_NET_HANDLE_MAXSIZE, child.stderr.read()[-3000:]
        handle = C.create_string_buffer(bytes.fromhex(line), P.NCCL_NET_HANDLE_MAXSIZE)
        p.reconfigure(**{k: env[k] for k in keys})
        scomm, deadline = None, time.time() + 60
        while not scomm:
            rc, scomm = p.connect(1, handle)
            assert rc == P.ncclSuccess and time.time() < deadline
        total = sum(sizes)
        src = torch.from_numpy(np.random.default_rng(34).integers(1, 256, size=total, dtype=np.uint8)).cuda()
        rc, mh = p.regMr(scomm, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
        assert rc == P.ncclSuccess
        offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)

        def send(q):
            req = None
            while not req:                  # no request while the receive has not been posted
                rc, req = p.isend(scomm, src.data_ptr() + int(offs[q]), sizes[q], q, mh)
                assert rc == P.ncclSuccess and time.time() < deadline
            return req

        def finish(req):
            done = 0
            while not done:
                rc, done, _ = p.test(req)
                assert rc == P.ncclSuccess and time.time() < deadline

        finish(send(0))
        together = [send(q) for q in (1, 2, 3, 4)]      # all four matched before anything is tested: one wave
        for r in together:
            finish(r)
        rows, hdr = p.last_table(scomm)
        n = sum(sizes[1:5])
        exp, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=n, chunk_bytes=chunk,
                                           mode=ob.SCHED_RESET_OFFSETS, state=_state(sizes[0], sizes[0] // chunk))
        assert rows.size == exp.size == (n + chunk - 1) // chunk
        for f in ("src_off", "win_off", "len", "lane"):
            np.testing.assert_array_equal(rows[f], exp[f], err_msg=f)
        np.testing.assert_array_equal(hdr["lane_bytes"][:lanes], exp_h["lane_bytes"][:lanes])
        finish(send(5))
        assert child.stdout.readline().strip() == "receiver ok", child.stderr.read()[-3000:]
        assert p.deregMr(scomm, mh) == P.ncclSuccess and p.closeSend(scomm) == P.ncclSuccess
        child.stdin.write("closed\n")
        child.stdin.flush()
        _, err = child.communicate(timeout=60)
        assert child.returncode == 0, err[-3000:]
    finally:
        if child.poll() is None:
            child.kill()
        p.reconfigure(**{k: None for k in keys})
