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


# ---- refreshes across the process boundary ----------------------------------------------------------------------------
# A receiver that takes a plan: the request sizes, request numbers in front of which it waits for a line on its standard
# input (so that this process can change something first), and optionally credit rows that it sets with fl_net_set_credits
# in front of the refresh they are for.  It posts one receive at a time, so nothing is in flight at a refresh boundary.
_PLANNED_RECEIVER = r"""
import json, sys, time
import numpy as np
import torch
from fuselink_amd import plugin as P
plan = json.loads(sys.argv[1])
sizes, seed, gates, rows, cadence = plan["sizes"], plan["seed"], plan.get("gates", []), plan.get("rows"), plan.get("cadence", 8)
p = P.NetPlugin(8)
assert p.init() == P.ncclSuccess
rc, handle, lcomm = p.listen(0)
assert rc == P.ncclSuccess
sys.stdout.write(handle.raw.hex() + "\n"); sys.stdout.flush()
rcomm = None
deadline = time.time() + 90
while not rcomm:
    rc, rcomm = p.accept(lcomm)
    assert rc == P.ncclSuccess and time.time() < deadline
total = sum(sizes)
dst = torch.zeros(total + 64, dtype=torch.uint8, device="cuda")
rc, mh = p.regMr(rcomm, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
assert rc == P.ncclSuccess
off = 0
for q, n in enumerate(sizes):
    if q in gates:
        sys.stdout.write("at %d\n" % q); sys.stdout.flush()
        assert sys.stdin.readline().strip() == "go"
    if rows is not None and q % cadence == 0:
        p.set_credits(rows[(q // cadence) % len(rows)])
    req = None
    while not req:
        rc, req = p.irecv(rcomm, [dst.data_ptr() + off], [n], [q], [mh])
        assert rc == P.ncclSuccess and time.time() < deadline
    done = 0
    while not done:
        rc, done, got = p.test(req)
        assert rc == P.ncclSuccess and time.time() < deadline
    assert got == n, (q, got, n)
    off += n
st = p.comm_stats(rcomm)
assert st["refreshes"] == (len(sizes) + cadence - 1) // cadence, st
torch.cuda.synchronize()
exp = np.random.default_rng(seed).integers(1, 256, size=total, dtype=np.uint8)
back = dst.cpu().numpy()
assert np.array_equal(back[:total], exp), "received bytes differ from what was sent"
assert not back[total:].any(), "bytes behind the last request were touched"
print("receiver ok"); sys.stdout.flush()
if plan.get("orphan"):
    # one more receive, which the sender never answers: once the sender has closed its end the receive must fail, not hang,
    # and its request must be freed
    req = None
    while not req:
        rc, req = p.irecv(rcomm, [dst.data_ptr()], [4096], [len(sizes)], [mh])
        assert rc == P.ncclSuccess and time.time() < deadline
    rc = P.ncclSuccess
    while rc == P.ncclSuccess:
        rc, done, _ = p.test(req)
        assert not done and time.time() < deadline
    assert rc == P.ncclRemoteError, rc
    assert p.free_requests(rcomm) == 256
    print("orphan failed"); sys.stdout.flush()
sys.stdin.readline()                    # the sender has closed its comm
assert p.deregMr(rcomm, mh) == P.ncclSuccess
assert p.closeRecv(rcomm) == P.ncclSuccess and p.closeListen(lcomm) == P.ncclSuccess
"""


class _Planned:
    """The sending side of a planned run, in this process: connects to the child, sends request by request and hands every
    request's table (of its last wave) to the caller's check."""

    def __init__(self, env, plan):
        import ctypes as C
        self.env = dict(os.environ, NCCL_FUSELINK_WIRE="shm", PYTHONPATH=ROOT, **{k: str(v) for k, v in env.items()})
        self.keys = ["NCCL_FUSELINK_WIRE"] + [k for k in env]
        self.plan = plan
        self.child = subprocess.Popen([sys.executable, "-c", _PLANNED_RECEIVER, json.dumps(plan)], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                                      stderr=subprocess.PIPE, text=True, env=self.env, cwd=ROOT)
        self.p = P.NetPlugin(8)
        self.C = C

    def __enter__(self):
        import torch
        line = self.child.stdout.readline().strip()
        assert len(line) == 2 * P.NCCL_NET_HANDLE_MAXSIZE, self.child.stderr.read()[-3000:]
        handle = self.C.create_string_buffer(bytes.fromhex(line), P.NCCL_NET_HANDLE_MAXSIZE)
        self.p.reconfigure(**{k: self.env[k] for k in self.keys})
        self.scomm, self.deadline = None, time.time() + 90
        while not self.scomm:
            rc, self.scomm = self.p.connect(1, handle)
            assert rc == P.ncclSuccess and time.time() < self.deadline
        sizes = self.plan["sizes"]
        self.src = torch.from_numpy(np.random.default_rng(self.plan["seed"]).integers(1, 256, size=sum(sizes), dtype=np.uint8)).cuda()
        rc, self.mh = self.p.regMr(self.scomm, self.src.data_ptr(), self.src.numel(), P.NCCL_PTR_CUDA)
        assert rc == P.ncclSuccess
        self.off = 0
        return self

    def gate(self, q):
        """The child stands in front of request q; returns once it says so (call release() to let it go on)."""
        line = self.child.stdout.readline().strip()
        assert line == f"at {q}", (line, self.child.stderr.read()[-3000:] if self.child.poll() is not None else "")

    def release(self):
        self.child.stdin.write("go\n")
        self.child.stdin.flush()

    def send(self, q):
        n = self.plan["sizes"][q]
        req = None
        while not req:                      # no request while the receive has not been posted
            rc, req = self.p.isend(self.scomm, self.src.data_ptr() + self.off, n, q, self.mh)
            assert rc == P.ncclSuccess and time.time() < self.deadline, self.child.stderr.read()[-3000:] if self.child.poll() is not None else "timed out"
        done = 0
        while not done:
            rc, done, _ = self.p.test(req)
            assert rc == P.ncclSuccess and time.time() < self.deadline
        self.off += n
        return self.p.last_table(self.scomm)

    def __exit__(self, et, ev, tb):
        try:
            if et is None:
                assert self.child.stdout.readline().strip() == "receiver ok", self.child.stderr.read()[-3000:]
                assert self.p.deregMr(self.scomm, self.mh) == P.ncclSuccess and self.p.closeSend(self.scomm) == P.ncclSuccess
                if self.plan.get("orphan"):
                    assert self.child.stdout.readline().strip() == "orphan failed", self.child.stderr.read()[-3000:]
                self.child.stdin.write("closed\n")
                self.child.stdin.flush()
                _, err = self.child.communicate(timeout=60)
                assert self.child.returncode == 0, err[-3000:]
        finally:
            if self.child.poll() is None:
                self.child.kill()
            if et is not None:
                try:
                    self.p.closeSend(self.scomm)
                except Exception:
                    pass
            self.p.reconfigure(**{k: None for k in self.keys})
        return False


def _check_last_wave(rows, n, credits, lanes, chunk, window_bytes, epoch, chunks_before, what):
    exp_all, _, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=n, chunk_bytes=chunk,
                                       mode=ob.SCHED_RESET_OFFSETS, state=_state(epoch, chunks_before))
    first = _waves(exp_all, lanes, window_bytes, chunk)[-1]
    at = int(exp_all["src_off"][first])
    exp, _, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=n - at, chunk_bytes=chunk, src_base=at,
                                   mode=ob.SCHED_RESET_OFFSETS, state=_state(epoch + at, chunks_before + first))
    assert rows.size == exp.size, (what, rows.size, exp.size)
    for f in ("src_off", "win_off", "len", "lane"):
        np.testing.assert_array_equal(rows[f], exp[f], err_msg=f"{what}, {f}")


@DIRECT
def test_refreshes_with_new_credit_rows_across_two_processes(direct):
    """The credit row travels in the descriptor, the epoch flag beside it.  With a cadence of 3 the receiving process
    sets a new row in front of every refresh; every request's table on the sending side must be the oracle's under the row
    its descriptor carried, from an epoch prefix that starts again at zero with every refresh.  Ragged requests and
    requests of several waves (2 MiB windows) among them."""
    lanes, chunk, cadence = 4, 128 << 10, 3
    rng = np.random.default_rng(77)
    rows = [[int(x) for x in rng.integers(0, 5, size=lanes)] for _ in range(5)]
    for r in rows:
        if sum(r) == 0:
            r[1] = 2
    sizes = [3 * chunk, 5 * chunk + 17, 20 << 20, chunk, 9 * chunk, (6 << 20) + 4321, 2 * chunk, 7 * chunk - 5, 4 * chunk, 11 * chunk + 1, chunk, 3 * chunk, 2 * chunk + 9]
    plan = dict(sizes=sizes, seed=78, rows=rows, cadence=cadence)
    env = {"NCCL_FUSELINK_LANES": lanes, "NCCL_FUSELINK_CHUNKSIZE": chunk, "NCCL_FUSELINK_WINDOW_UNITS": 1, "NCCL_FUSELINK_ENGINE_UNITS": 1,
           "NCCL_FUSELINK_REFRESH_BATCH": cadence, "NCCL_FUSELINK_WIRE_DIRECT": direct}
    with _Planned(env, plan) as run:
        epoch = chunks = 0
        for q, n in enumerate(sizes):
            if q % cadence == 0:
                epoch = 0                    # the descriptor said: refreshed
            table, hdr = run.send(q)
            _check_last_wave(table, n, rows[(q // cadence) % len(rows)], lanes, chunk, 2 << 20, epoch, chunks, f"request {q}")
            epoch += n
            chunks += (n + chunk - 1) // chunk
        assert run.p.mask_stats(run.scomm)["refreshes"] == sum(1 for k in range(len(sizes)) if (k + 1) % cadence == 0)


def _third_party_sets(shm, sem, lane, is_tx, status, stamp_in_us):
    """Another process writes one entry of the shared lane table, as anything that maps the reference's shared memory can."""
    code = ("import sys; from fuselink_amd import plugin as P; p = P.NetPlugin(8); L = p.lib; "
            f"assert L.fl_monitor_attach_shm({shm!r}, {sem!r}, 0) == 0; "
            f"assert L.fl_monitor_set_entry({lane}, {is_tx}, {status}, L.fl_monitor_now() + {stamp_in_us}) == 0; L.fl_monitor_detach()")
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=ROOT, env=dict(os.environ, PYTHONPATH=ROOT), timeout=120)
    assert res.returncode == 0, res.stderr[-2000:]


def test_a_lane_that_another_process_keeps_busy_gets_no_chunks_after_the_next_refresh():
    """FuseLink's point, end to end: the monitor daemon owns the lane table in shared memory; the sending and the receiving
    process both read it (NCCL_FUSELINK_MONITOR_SHM=1) and refresh on the reference's cadence of 8.  A third process marks
    the receive side of lane 5 BUSY; from the receiver's next refresh on, no chunk of any request lands on lane 5 and the
    sender's tables are the oracle's under the row fl_rx_credits_from_status gives for the table as it stands.  The third
    process lets the lane go; after the following refresh it carries chunks again."""
    from fuselink_amd import build as B
    import ctypes as C
    exe = B.monitor_path()
    if not os.path.exists(exe):
        pytest.skip("fuselink-monitor is not built")
    lanes, chunk, idle = 8, 64 << 10, 4
    daemon = subprocess.Popen([exe, "--seconds", "120"], stdout=subprocess.PIPE, text=True)     # the reference's names: /rdma_monitor_shm, /rdma_monitor_sem
    try:
        assert "table up" in daemon.stdout.readline()
        sizes = [6 * chunk + (q % 3) for q in range(24)]
        plan = dict(sizes=sizes, seed=91, gates=[8, 16])
        env = {"NCCL_FUSELINK_LANES": lanes, "NCCL_FUSELINK_CHUNKSIZE": chunk, "NCCL_FUSELINK_MONITOR_SHM": 1, "NCCL_FUSELINK_IDLE_CREDIT": idle}
        O = ob.lib()

        def expected_row(busy_rx):
            st = (C.c_int32 * lanes)(*[1 if l in busy_rx else 0 for l in range(lanes)])
            out = (C.c_uint32 * lanes)()
            O.fl_rx_credits_from_status(st, lanes, 0, idle, 0xffffffff, out)      # the receiving comm listens on lane 0
            return list(out)

        with _Planned(env, plan) as run:
            run.p.set_credits([])                # (no static row left over from another test)
            epoch = chunks = 0
            on_lane = [0, 0, 0]
            row = expected_row([])
            for q, n in enumerate(sizes):
                if q in (8, 16):
                    run.gate(q)
                    if q == 8:
                        _third_party_sets(None, None, 5, 0, 1, 60_000_000)       # BUSY, stamped a minute ahead: the daemon keeps it so
                    else:
                        _third_party_sets(None, None, 5, 0, 0, 0)                # IDLE again
                    time.sleep(0.01)                                              # (the lanes this traffic stamped age out: 160 us)
                    row = expected_row([5] if q == 8 else [])
                    run.release()
                if q % 8 == 0:
                    epoch = 0
                table, hdr = run.send(q)
                if 8 <= q < 16:
                    assert hdr["lane_chunks"][5] == 0 and 5 not in set(table["lane"].tolist()), f"request {q} put chunks on the busy lane"
                else:
                    on_lane[q // 8] += int(hdr["lane_chunks"][5])
                _check_last_wave(table, n, row, lanes, chunk, 8 << 20, epoch, chunks, f"request {q}")
                epoch += n
                chunks += (n + chunk - 1) // chunk
            assert on_lane[0] > 0 and on_lane[2] > 0      # before, and again after
            assert expected_row([5])[5] == 0 and expected_row([])[5] == idle
    finally:
        daemon.send_signal(15)
        daemon.wait(timeout=10)


def test_a_lane_that_the_senders_process_masks_out_gets_no_chunks_after_the_next_refresh():
    """The other half of the decision: what the SENDER knows.  No shared table here -- each process keeps its own -- so the
    only way the receiver can learn that the sender's lane 3 is busy is the mask in the immediate data.  This process marks
    the send side of lane 3 BUSY in front of the send at which its mask is refreshed ((n_finished + 1) % 8 == 0); the
    receiver keeps the mask of the completed receive and ANDs it into its row at its next refresh: requests 8 to 15 put
    nothing on lane 3.  The mark is taken away before the next refresh of the mask; from request 16 on lane 3 is back."""
    import ctypes as C
    lanes, chunk, idle = 8, 64 << 10, 4
    sizes = [5 * chunk + (q % 2) for q in range(24)]
    plan = dict(sizes=sizes, seed=92, gates=[8, 16])
    env = {"NCCL_FUSELINK_LANES": lanes, "NCCL_FUSELINK_CHUNKSIZE": chunk, "NCCL_FUSELINK_IDLE_CREDIT": idle}
    O = ob.lib()

    def expected_row(mask):
        st = (C.c_int32 * lanes)()
        out = (C.c_uint32 * lanes)()
        O.fl_rx_credits_from_status(st, lanes, 0, idle, mask, out)
        return list(out)

    with _Planned(env, plan) as run:
        L = run.p.lib
        L.fl_monitor_reset()
        run.p.set_credits([])                    # (no static row left over from another test: the mask comes off the lane table)
        epoch = chunks = 0
        on_lane = [0, 0, 0]
        row = expected_row(0xffffffff)
        for q, n in enumerate(sizes):
            if q == 6:
                assert L.fl_monitor_set_entry(3, 1, 1, L.fl_monitor_now() + 60_000_000) == 0     # lane 3's send side: BUSY for the next minute
            if q == 14:
                assert L.fl_monitor_set_entry(3, 1, 0, 0) == 0
            if q in (8, 16):
                run.gate(q)
                time.sleep(0.01)                                                                  # (the lanes this traffic stamped age out)
                mask = run.p.mask_stats(run.scomm)["mask"]
                assert mask == (0xfffffff7 if q == 8 else 0xffffffff), hex(mask)
                row = expected_row(mask)
                run.release()
            if q % 8 == 0:
                epoch = 0
            table, hdr = run.send(q)
            if 8 <= q < 16:
                assert hdr["lane_chunks"][3] == 0, f"request {q} put chunks on the lane the sender had masked out"
            else:
                on_lane[q // 8] += int(hdr["lane_chunks"][3])
            _check_last_wave(table, n, row, lanes, chunk, 8 << 20, epoch, chunks, f"request {q}")
            epoch += n
            chunks += (n + chunk - 1) // chunk
        assert on_lane[0] > 0 and on_lane[2] > 0          # before, and again after
        st = run.p.mask_stats(run.scomm)
        assert st["refreshes"] == 3 and st["mask"] == 0xffffffff
        L.fl_monitor_reset()


@DIRECT
def test_a_receive_whose_sender_has_gone_fails_and_is_freed(direct):
    """The other process closes its end with a receive still posted here: test returns ncclRemoteError for it (as a failed
    completion does, src/plugin.cc:1839-1861) instead of polling for ever, and the request goes back to the table.  And the
    other way round: a send that finds the receiving process gone fails at once."""
    lanes, chunk = 4, 128 << 10
    plan = dict(sizes=[3 * chunk, 5 * chunk + 7], seed=55, orphan=True)
    env = {"NCCL_FUSELINK_LANES": lanes, "NCCL_FUSELINK_CHUNKSIZE": chunk, "NCCL_FUSELINK_WIRE_DIRECT": direct}
    with _Planned(env, plan) as run:
        for q in range(len(plan["sizes"])):
            run.send(q)


@DIRECT
@pytest.mark.parametrize("seed", [11, 12])
def test_random_traffic_of_several_connections_both_ways_across_two_processes(direct, seed):
    """The reference's two ends both send and receive, on several channels at once.  Three connections from this process
    to the child and two back, 24 requests each from empty to 1.5 MiB (some whole chunks, some a few bytes, one of 7.5 MiB
    that the windows hold only in pieces), six in flight per connection, posted and tested in a seeded random order by
    both processes at once: requests of different connections share waves, waves of both directions share each GPU
    side's queue and engine, the refresh gate closes and opens on the default cadence.  Each process compares what it
    received with the connection's pattern, and the bytes behind it with zero."""
    from tests import two_process_peer as peer
    lanes, chunk = 4, 128 << 10
    env = dict(os.environ, NCCL_FUSELINK_WIRE="shm", PYTHONPATH=ROOT, NCCL_FUSELINK_LANES=str(lanes), NCCL_FUSELINK_CHUNKSIZE=str(chunk),
               NCCL_FUSELINK_WINDOW_UNITS="1", NCCL_FUSELINK_WIRE_DIRECT=str(direct))
    plan = peer.make_plan(seed, n_ab=3, n_ba=2, requests=24, max_bytes=3 << 19, chunk=chunk, inflight=6)
    child = subprocess.Popen([sys.executable, "-m", "tests.two_process_peer", json.dumps(plan)], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                             stderr=subprocess.PIPE, text=True, env=env, cwd=ROOT)
    keys = ["NCCL_FUSELINK_WIRE"] + list(env_keys(env))
    p = P.NetPlugin(8)

    def write_line(s):
        child.stdin.write(s + "\n")
        child.stdin.flush()

    try:
        p.reconfigure(**{k: env[k] for k in keys})
        p.set_credits([])                # no static row left by an earlier test: the monitor drives
        n = peer.drive(p, P, plan, "a", child.stdout.readline, write_line, peer_alive=lambda: child.poll() is None)
        assert n == sum(len(c["sizes"]) for c in plan["conns"])
        assert child.stdout.readline().strip() == f"peer ok {n}", child.stderr.read()[-3000:]
        _, err = child.communicate(timeout=60)
        assert child.returncode == 0, err[-3000:]
    except AssertionError:
        if child.poll() is None:
            child.kill()
        print(child.stderr.read()[-3000:])
        raise
    finally:
        if child.poll() is None:
            child.kill()
        p.reconfigure(**{k: None for k in keys})
