"""The lane engine (flh_engine_*): a resident kernel that executes batches from a descriptor ring instead of from a launch
pair each.  What it stages and delivers must be what flh_stripe_batch / flh_reassemble_batch stage and deliver, i.e. the
oracle's tables and bytes; it must go down when idle and come up again with the next batch; bad arguments are refused on
the host."""
import ctypes as C
import time

import numpy as np
import pytest

from tests import oracle_binding as ob

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fl():
    import torch
    from fuselink_amd import _lib, core
    core.init(0)
    return core, torch, _lib


def _dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _wait(lib, eng, seq, seconds=10.0):
    deadline = time.time() + seconds
    while lib.flh_engine_completed(eng) < seq:
        assert lib.flh_engine_error(eng) == 0, "the engine reported a wait that ran out"
        if lib.flh_engine_needs_start(eng):      # its time as a resident ran out between two batches: whoever waits starts the next one
            assert lib.flh_engine_poke(eng) == 0
        assert time.time() < deadline, f"batch {seq} did not complete (completed {lib.flh_engine_completed(eng)})"


@pytest.mark.parametrize("sets", [1, 2, 3, 8])
def test_engine_batches_equal_the_oracle_and_the_engine_restarts_after_idling(fl, sets):
    core, torch, _lib = fl
    lib = _lib.load()
    rng = np.random.default_rng(7300 + sets)
    lanes, chunk, n_batches = 6, 32 << 10, 7
    eng = C.c_void_p()
    _lib.check(lib.flh_engine_create(0, 0, 100, sets, C.byref(eng)))     # idle limit 100 us
    _lib.check(lib.flh_engine_set_resident(eng, 0))                      # (the launches are counted below: only idling takes it down)
    try:
        cap = 3 << 20
        wins = [[torch.zeros(cap + 64, dtype=torch.uint8, device="cuda") for _ in range(lanes)] for _ in range(sets)]
        W = [core.make_windows([t.data_ptr() for t in ws], [cap] * lanes) for ws in wins]
        status = core.new_status()
        batches = []
        for k in range(n_batches):
            n_seg = int(rng.integers(1, 4))
            segments, sizes = [], []
            for _ in range(n_seg):
                n_req = int(rng.integers(1, 5))
                ss = [int(rng.integers(1, 6)) * chunk for _ in range(n_req)]
                if rng.random() < 0.5:
                    ss[-1] -= int(rng.integers(1, chunk))
                segments.append((n_req, rng.integers(0, 6, size=lanes).astype(np.uint32), int(rng.integers(0, 30)) * chunk))
                sizes += ss
            srcs_np = [rng.integers(0, 256, size=s, dtype=np.uint8) for s in sizes]
            srcs = [_dev(torch, a) for a in srcs_np]
            dsts = [torch.zeros(s + 32, dtype=torch.uint8, device="cuda") for s in sizes]
            n_rows = sum((s + chunk - 1) // chunk for s in sizes) + len(segments)
            batches.append(dict(segments=segments, sizes=sizes, srcs_np=srcs_np, srcs=srcs, dsts=dsts, out=core.new_schedule_buffers(n_rows)))
        torch.cuda.synchronize()
        seq = C.c_uint64()
        for k, bt in enumerate(batches):
            b = core.batch_params(bt["srcs"], bt["dsts"], chunk, [1] * lanes, segments=[(n, c.tolist(), e) for n, c, e in bt["segments"]])
            _lib.check(lib.flh_engine_submit(eng, C.byref(b), C.byref(W[k % sets]), bt["out"].table.data_ptr(), bt["out"].hdr.data_ptr(),
                                             status.data_ptr(), C.byref(seq), None))
            assert seq.value == k + 1
            if k == 2:
                _wait(lib, eng, seq.value)
                time.sleep(0.02)            # far beyond the idle limit: the engine goes down, the next submit starts it again
                assert int(lib.flh_engine_launches(eng)) == 1
            if sets == 1:
                _wait(lib, eng, seq.value)  # one window set: the caller may not have two batches in flight
        _wait(lib, eng, seq.value)
        assert int(lib.flh_engine_launches(eng)) == 2 and lib.flh_engine_error(eng) == 0
        torch.cuda.synchronize()
        assert int(status.item()) == 0
        for k, bt in enumerate(batches):
            lane_end = np.zeros(16, dtype=np.uint64)
            rows, first_row, q = [], 0, 0
            tpc = (chunk + 32767) // 32768
            staged = []
            for n_req, credits, epoch in bt["segments"]:
                seg_np = np.concatenate(bt["srcs_np"][q:q + n_req])
                q += n_req
                st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
                st["epoch_bytes"] = epoch
                exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=seg_np.size, chunk_bytes=chunk,
                                                     mode=ob.SCHED_RESET_OFFSETS, state=st)
                base = (lane_end + np.uint64(127)) // np.uint64(128) * np.uint64(128)
                wins_seg = ob.cpu_stripe(seg_np, exp_t, [int(x) for x in exp_h["lane_bytes"][:lanes]])
                for l in range(lanes):
                    n = int(exp_h["lane_bytes"][l])
                    if n:
                        staged.append((l, int(base[l]), wins_seg[l][:n]))
                r = exp_t.copy()
                r["win_off"] += base[r["lane"]]
                r["tile_base"] += first_row * tpc
                rows.append(r)
                used = exp_h["lane_chunks"] > 0
                lane_end[used] = base[used] + exp_h["lane_bytes"][used]
                first_row += len(exp_t)
            exp_rows = np.concatenate(rows)
            bt["out"].n_chunks = len(exp_rows)
            got = bt["out"].table_numpy()
            for f in ob.DESC_DTYPE.names:
                np.testing.assert_array_equal(got[f], exp_rows[f], err_msg=f"batch {k}: {f}")
            assert int(bt["out"].hdr_numpy()["n_chunks"]) == len(exp_rows)
            if k >= n_batches - sets:       # the window sets still hold what their last batch staged
                for l, off, data in staged:
                    np.testing.assert_array_equal(wins[k % sets][l].cpu().numpy()[off:off + data.size], data, err_msg=f"batch {k} lane {l}")
            for i, s in enumerate(bt["sizes"]):
                g = bt["dsts"][i].cpu().numpy()
                np.testing.assert_array_equal(g[:s], bt["srcs_np"][i], err_msg=f"batch {k} request {i}")
                assert not g[s:].any()
    finally:
        _lib.check(lib.flh_engine_destroy(eng))


def test_buffers_that_are_used_again_deliver_their_latest_contents(fl):
    """The workers stay resident, so no kernel boundary brings their view of memory up to date or makes their stores
    visible: they must read what a kernel on another stream has just written into a source they have read before, and a
    kernel that starts once a batch is complete must read what they delivered.  The same sources, windows and
    destinations carry new contents in each of 48 batches (sizes that end in odd bytes among them, so the byte edges
    and the shifted copy take part); every destination is compared on the GPU, by a kernel, not through a DMA copy.
    Half-way the batches go two at a time, alternating between two sets of buffers."""
    core, torch, _lib = fl
    lib = _lib.load()
    lanes, chunk, sets = 8, 64 << 10, 2
    sizes = [512 << 10, (512 << 10) - 7, 100_003, 64 << 10, 33]
    eng = C.c_void_p()
    _lib.check(lib.flh_engine_create(0, 0, 200, sets, C.byref(eng)))
    try:
        cap = 2 << 20
        wins = [[torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)] for _ in range(sets)]
        W = [core.make_windows([t.data_ptr() for t in ws], [cap] * lanes) for ws in wins]
        status = core.new_status()
        bufs = []
        for _ in range(sets):
            srcs = [torch.zeros(n, dtype=torch.uint8, device="cuda") for n in sizes]
            dsts = [torch.zeros(n + 64, dtype=torch.uint8, device="cuda") for n in sizes]
            # only a segment's last request may end inside a chunk: three segments, each with a credit row of its own
            segments = [(2, [3, 1, 2, 1, 1, 2, 1, 1], 0), (1, [1, 1, 1, 1, 0, 0, 2, 2], 3 * chunk), (2, [1] * lanes, 0)]
            bufs.append((srcs, dsts, core.batch_params(srcs, dsts, chunk, [1] * lanes, segments=segments)))
        gen = torch.Generator(device="cuda")
        gen.manual_seed(4711)
        seq = C.c_uint64()

        def refill(which):
            for t in bufs[which][0]:
                t.copy_(torch.randint(0, 256, t.shape, dtype=torch.uint8, device="cuda", generator=gen))
            for t in bufs[which][1]:
                t.fill_(0xEE)

        def submit(which):
            _lib.check(lib.flh_engine_submit(eng, C.byref(bufs[which][2]), C.byref(W[which]), None, None, status.data_ptr(), C.byref(seq), None))
            return seq.value

        def check(which, k):
            for i, n in enumerate(sizes):
                src, dst = bufs[which][0][i], bufs[which][1][i]
                assert bool(torch.equal(dst[:n], src)), f"batch {k}, request {i}: stale or missing bytes"
                assert bool((dst[n:] == 0xEE).all()), f"batch {k}, request {i}: bytes past the end"

        for k in range(24):                 # one at a time, the same buffers every time
            refill(0)
            torch.cuda.synchronize()        # the contract of a submit: what it reads has been written
            _wait(lib, eng, submit(0))
            check(0, k)
        for k in range(24, 48, 2):          # two in flight
            refill(0)
            refill(1)
            torch.cuda.synchronize()
            submit(0)
            _wait(lib, eng, submit(1))
            check(0, k)
            check(1, k + 1)
        torch.cuda.synchronize()
        assert int(status.item()) == 0 and lib.flh_engine_error(eng) == 0
    finally:
        _lib.check(lib.flh_engine_destroy(eng))


def test_engine_refuses_bad_arguments_on_the_host(fl):
    core, torch, _lib = fl
    lib = _lib.load()
    eng = C.c_void_p()
    assert lib.flh_engine_create(0, 0, 0, 0, C.byref(eng)) == -1       # no window set
    assert lib.flh_engine_create(0, 0, 0, 9, C.byref(eng)) == -1       # more sets than the engine keeps descriptors for
    assert lib.flh_engine_create(0, 1, 0, 2, C.byref(eng)) == -1       # a dispatcher without workers
    _lib.check(lib.flh_engine_create(0, 9, 0, 2, C.byref(eng)))
    try:
        chunk = 4096
        srcs = [torch.zeros(chunk + 1, dtype=torch.uint8, device="cuda"), torch.zeros(chunk, dtype=torch.uint8, device="cuda")]
        dsts = [torch.zeros_like(t) for t in srcs]
        wins = [torch.zeros(8 * chunk, dtype=torch.uint8, device="cuda") for _ in range(2)]
        w = core.make_windows([t.data_ptr() for t in wins], [8 * chunk] * 2)
        out = core.new_schedule_buffers(8)
        status = core.new_status()
        seq = C.c_uint64()
        b = core.batch_params(srcs, dsts, chunk, [1, 1])
        with pytest.raises(Exception, match="whole number of chunks"):
            _lib.check(lib.flh_engine_submit(eng, C.byref(b), C.byref(w), out.table.data_ptr(), out.hdr.data_ptr(), status.data_ptr(), C.byref(seq), None))
        assert int(lib.flh_engine_launches(eng)) == 0 and int(lib.flh_engine_completed(eng)) == 0
    finally:
        _lib.check(lib.flh_engine_destroy(eng))


@pytest.mark.gpu
def test_engine_harness_moves_the_bytes_and_reports_its_latency():
    """tests/harness/engine_bench drives flh_engine_* from C++ the way the plugin does (a batch at a time, several in
    flight, after the engine has gone down for lack of work) and compares what arrived with what was sent."""
    import json
    import os
    import subprocess
    from fuselink_amd import build
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "harness", "engine_bench")
    if not os.path.exists(exe):
        build.build_harness(verbose=False)
    res = subprocess.run([exe, build.lib_path(), "--requests", "5", "--depth", "3", "--batches", "300"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr[-2000:]
    out = json.loads(res.stdout.strip().splitlines()[-1])
    assert out["bit_exact"] and out["requests_per_batch"] == 5 and out["engine_launches"] >= 20   # every idle period took it down
    assert 0 < out["in_flight_us_per_batch"] <= out["one_at_a_time_us_per_batch"] * 1.2
    print(out)


def test_a_wait_that_runs_out_takes_the_engine_down_and_is_reported(fl):
    """Every wait inside the resident kernel is bounded.  With the bound set to a microsecond and one window set, the
    workers of a second batch cannot get the windows before the first batch is through: their wait runs out, the kernel
    reports FLH_E_STATE through the control block and every workgroup leaves (the stream drains, destroy returns);
    later submits are refused.  No kernel is left spinning."""
    core, torch, _lib = fl
    lib = _lib.load()
    lanes, chunk, n_req = 8, 256 << 10, 32
    _lib.check(lib.flh_tune(b"engine_wait_us", 1))
    eng = C.c_void_p()
    try:
        _lib.check(lib.flh_engine_create(0, 0, 100000, 1, C.byref(eng)))
    finally:
        _lib.check(lib.flh_tune(b"engine_wait_us", 2000000))
    try:
        cap = 8 << 20
        wins = [torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
        W = core.make_windows([t.data_ptr() for t in wins], [cap] * lanes)
        status = core.new_status()
        srcs = [torch.full((512 << 10,), 1 + q, dtype=torch.uint8, device="cuda") for q in range(n_req)]
        dsts = [torch.zeros(512 << 10, dtype=torch.uint8, device="cuda") for _ in range(n_req)]
        out = core.new_schedule_buffers(n_req * 2 + 1)
        b = core.batch_params(srcs, dsts, chunk, [1] * lanes)
        torch.cuda.synchronize()
        seq = C.c_uint64()
        for _ in range(2):   # back to back: the second batch wants the first one's windows
            _lib.check(lib.flh_engine_submit(eng, C.byref(b), C.byref(W), out.table.data_ptr(), out.hdr.data_ptr(), status.data_ptr(), C.byref(seq), None))
        deadline = time.time() + 10
        while lib.flh_engine_error(eng) == 0 and lib.flh_engine_completed(eng) < 2:
            assert time.time() < deadline, "neither an error nor completion"
        assert lib.flh_engine_error(eng) == -6    # FLH_E_STATE: an error, not completion
        assert lib.flh_engine_completed(eng) < 2
        rc = lib.flh_engine_submit(eng, C.byref(b), C.byref(W), out.table.data_ptr(), out.hdr.data_ptr(), status.data_ptr(), C.byref(seq), None)
        assert rc < 0 and b"went down" in lib.flh_last_error()
    finally:
        t0 = time.time()
        _lib.check(lib.flh_engine_destroy(eng))     # waits for the kernel: it has left, or leaves at its next poll
        assert time.time() - t0 < 5
        torch.cuda.synchronize()


def test_the_engine_stamps_the_stages_of_its_batches_when_asked(fl):
    """Measurement: an engine created while flh_tune("engine_trace") is set stamps every batch's stages with the GPU's wall
    clock (dispatcher saw the tail, published, first worker saw it, was let in, had the descriptor, had moved its shares,
    completion word acknowledged).  Stamps of a batch never run backwards, a batch's whole stay in the kernel is
    microseconds, and an engine created without the switch refuses the call."""
    core, torch, _lib = fl
    lib = _lib.load()
    lib.flh_tune.argtypes = [C.c_char_p, C.c_int64]
    lanes, chunk, n = 4, 64 << 10, 12
    plain = C.c_void_p()
    _lib.check(lib.flh_engine_create(0, 0, 200, 2, C.byref(plain)))
    assert lib.flh_tune(b"engine_trace", 1) == 0
    eng = C.c_void_p()
    try:
        _lib.check(lib.flh_engine_create(0, 0, 200, 2, C.byref(eng)))
    finally:
        assert lib.flh_tune(b"engine_trace", 0) == 0
    try:
        cap = 1 << 20
        wins = [[torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)] for _ in range(2)]
        W = [core.make_windows([t.data_ptr() for t in ws], [cap] * lanes) for ws in wins]
        status = core.new_status()
        src_np = np.random.default_rng(5).integers(0, 256, size=6 * chunk + 100, dtype=np.uint8)
        src = _dev(torch, src_np)
        dsts = [torch.zeros(src_np.size, dtype=torch.uint8, device="cuda") for _ in range(n)]
        out = core.new_schedule_buffers(8)
        torch.cuda.synchronize()
        seq = C.c_uint64()
        for k in range(n):
            b = core.batch_params([src], [dsts[k]], chunk, [2, 1, 1, 3])
            _lib.check(lib.flh_engine_submit(eng, C.byref(b), C.byref(W[k % 2]), out.table.data_ptr(), out.hdr.data_ptr(), status.data_ptr(), C.byref(seq), None))
            _wait(lib, eng, seq.value)
        stamps = (C.c_uint64 * (7 * n))()
        _lib.check(lib.flh_engine_trace(eng, 1, n, stamps))
        st = np.frombuffer(stamps, dtype=np.uint64).reshape(n, 7).astype(np.int64)
        assert (st > 0).all()
        assert (np.diff(st, axis=1) >= 0).all(), st
        assert ((st[:, -1] - st[:, 0]) < 100 * 1000).all()          # under a millisecond of the 100 MHz clock
        assert (np.diff(st[:, 0]) > 0).all()                        # batch after batch
        assert lib.flh_engine_trace(eng, 1, n + 1, stamps) != 0      # not complete yet
        assert lib.flh_engine_trace(plain, 1, 1, stamps) != 0        # keeps no trace
        torch.cuda.synchronize()
        for k in range(n):
            np.testing.assert_array_equal(dsts[k].cpu().numpy(), src_np)
    finally:
        _lib.check(lib.flh_engine_destroy(eng))
        _lib.check(lib.flh_engine_destroy(plain))
