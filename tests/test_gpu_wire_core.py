"""The two halves of a transfer whose ends are different processes, at the level of the C ABI: the striping launch that
carries every staged tile on into the receiver's landing windows (flh_stripe_uniform_carry / flh_stripe_batch_carry: staging
plus the wire, the part a NIC per lane plays in FuseLink src/plugin.cc:1453-1495), the engine batches that do the same
without a launch (FLH_ENGINE_SEND) and that deliver out of landing windows (FLH_ENGINE_RECV), and the engine's housekeeping
around them: a bounded time as a resident, a submit whose failure is final.  Tables, staged bytes, landed bytes and delivered
bytes are the oracle's."""
import ctypes as C
import time

import numpy as np
import pytest

from tests import oracle_binding as ob

pytestmark = pytest.mark.gpu

SEND, RECV = 1, 2


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
        if lib.flh_engine_needs_start(eng):
            assert lib.flh_engine_poke(eng) == 0
        assert time.time() < deadline, f"batch {seq} did not complete (completed {lib.flh_engine_completed(eng)})"


def _state(epoch_bytes):
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["epoch_bytes"] = epoch_bytes
    return st


def _expect_batch(segments, srcs_np, lanes, chunk):
    """Rows of the batch's table and what every lane's window holds ((lane, offset, bytes) triples), from the oracle run
    segment by segment, each segment behind the ones before it at the next multiple of 128 bytes."""
    lane_end = np.zeros(16, dtype=np.uint64)
    rows, staged, first_row, q = [], [], 0, 0
    tpc = (chunk + 32767) // 32768
    for n_req, credits, epoch in segments:
        seg_np = np.concatenate(srcs_np[q:q + n_req])
        q += n_req
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=np.asarray(credits, dtype=np.uint32), quantum=chunk, total_bytes=seg_np.size,
                                             chunk_bytes=chunk, mode=ob.SCHED_RESET_OFFSETS, state=_state(epoch))
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
    return np.concatenate(rows), staged


@pytest.mark.parametrize("nbytes,chunk,lanes,epoch_chunks", [((4 << 20) + 4096 + 3, 256 << 10, 8, 0), (64 << 20, 256 << 10, 8, 5), (7 * (96 << 10) + 1, 96 << 10, 3, 2)])
def test_a_striping_launch_with_a_carry_lands_the_oracles_windows(fl, nbytes, chunk, lanes, epoch_chunks):
    core, torch, _lib = fl
    lib = _lib.load()
    rng = np.random.default_rng(nbytes % 9973 + lanes)
    credits = rng.integers(1, 9, size=lanes).astype(np.uint32)
    epoch = epoch_chunks * chunk
    src_np = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=nbytes, chunk_bytes=chunk,
                                         mode=ob.SCHED_RESET_OFFSETS, state=_state(epoch))
    lane_bytes = [int(x) for x in exp_h["lane_bytes"][:lanes]]
    exp_w = ob.cpu_stripe(src_np, exp_t, lane_bytes)
    src = _dev(torch, src_np)
    dst = torch.zeros(nbytes + 64, dtype=torch.uint8, device="cuda")
    stage = [torch.zeros(max(b, 1) + 64, dtype=torch.uint8, device="cuda") for b in lane_bytes]
    land = [torch.full((max(b, 1) + 64,), 0xEE, dtype=torch.uint8, device="cuda") for b in lane_bytes]
    W = core.make_windows([t.data_ptr() for t in stage], lane_bytes)
    L = core.make_windows([t.data_ptr() for t in land], lane_bytes)
    status = core.new_status()
    out = core.new_schedule_buffers(len(exp_t))
    u = core.uniform_params(nbytes, chunk, credits.tolist(), epoch_bytes=epoch)
    # the launch reports itself: it is the last of the path on the sending side
    done = torch.zeros(64, dtype=torch.int32).pin_memory()
    count = torch.zeros(64, dtype=torch.int32, device="cuda")
    if nbytes < (8 << 20):
        u.d_done_word, u.d_done_count, u.done_value = done.data_ptr(), count.data_ptr(), 41
    _lib.check(lib.flh_stripe_uniform_carry(src.data_ptr(), nbytes, C.byref(W), C.byref(L), C.byref(u), out.table.data_ptr(), out.hdr.data_ptr(),
                                            status.data_ptr(), None))
    if nbytes < (8 << 20):
        deadline = time.time() + 10
        while int(done[0]) != 41:
            assert time.time() < deadline, "the completion word never came"
    u.d_done_word = u.d_done_count = None
    core.reassemble_uniform(dst, L, u, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and int(count[0].item()) == 0
    got = out.table_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got[f], exp_t[f], err_msg=f)
    for l in range(lanes):
        np.testing.assert_array_equal(stage[l].cpu().numpy()[:lane_bytes[l]], exp_w[l][:lane_bytes[l]], err_msg=f"staging window {l}")
        g = land[l].cpu().numpy()
        np.testing.assert_array_equal(g[:lane_bytes[l]], exp_w[l][:lane_bytes[l]], err_msg=f"landing window {l}")
        assert (g[lane_bytes[l]:] == 0xEE).all(), f"landing window {l}: bytes behind the lane's share were touched"
    back = dst.cpu().numpy()
    np.testing.assert_array_equal(back[:nbytes], src_np)
    assert not back[nbytes:].any()


def test_a_carry_that_would_leave_its_landing_window_is_refused(fl):
    core, torch, _lib = fl
    lib = _lib.load()
    lanes, chunk, nbytes = 2, 64 << 10, 8 * (64 << 10)
    src = torch.ones(nbytes, dtype=torch.uint8, device="cuda")
    stage = [torch.zeros(4 * chunk, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
    land = [torch.zeros(4 * chunk, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
    W = core.make_windows([t.data_ptr() for t in stage], [4 * chunk] * lanes)
    L = core.make_windows([t.data_ptr() for t in land], [4 * chunk, 3 * chunk])      # lane 1 lands one chunk short
    status = core.new_status()
    u = core.uniform_params(nbytes, chunk, [1, 1])
    _lib.check(lib.flh_stripe_uniform_carry(src.data_ptr(), nbytes, C.byref(W), C.byref(L), C.byref(u), None, None, status.data_ptr(), None))
    torch.cuda.synchronize()
    assert int(status.item()) == -5                                                   # FLH_E_RANGE
    assert land[1].cpu().numpy()[:3 * chunk].all() and land[0].cpu().numpy().all()    # what fitted landed; nothing beyond was written
    Lbad = core.make_windows([t.data_ptr() for t in land[:1]], [4 * chunk])
    assert lib.flh_stripe_uniform_carry(src.data_ptr(), nbytes, C.byref(W), C.byref(Lbad), C.byref(u), None, None, status.data_ptr(), None) == -1
    assert lib.flh_stripe_uniform_carry(src.data_ptr(), nbytes, C.byref(W), None, C.byref(u), None, None, status.data_ptr(), None) == -1


def _random_batch(rng, torch, lanes, chunk, max_seg=3, max_req=4):
    n_seg = int(rng.integers(1, max_seg + 1))
    segments, sizes = [], []
    for _ in range(n_seg):
        n_req = int(rng.integers(1, max_req + 1))
        ss = [int(rng.integers(1, 6)) * chunk for _ in range(n_req)]
        if rng.random() < 0.5:
            ss[-1] -= int(rng.integers(1, chunk))
        segments.append((n_req, rng.integers(0, 6, size=lanes).astype(np.uint32).tolist(), int(rng.integers(0, 30)) * chunk))
        sizes += ss
    srcs_np = [rng.integers(0, 256, size=s, dtype=np.uint8) for s in sizes]
    return dict(segments=segments, sizes=sizes, srcs_np=srcs_np, srcs=[_dev(torch, a) for a in srcs_np],
                dsts=[torch.zeros(s + 32, dtype=torch.uint8, device="cuda") for s in sizes])


def test_a_batch_launch_with_a_carry_lands_what_the_batch_stages(fl):
    core, torch, _lib = fl
    lib = _lib.load()
    rng = np.random.default_rng(811)
    lanes, chunk, cap = 5, 32 << 10, 3 << 20
    for _ in range(4):
        bt = _random_batch(rng, torch, lanes, chunk)
        stage = [torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
        land = [torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
        W = core.make_windows([t.data_ptr() for t in stage], [cap] * lanes)
        L = core.make_windows([t.data_ptr() for t in land], [cap] * lanes)
        status = core.new_status()
        exp_rows, staged = _expect_batch(bt["segments"], bt["srcs_np"], lanes, chunk)
        out = core.new_schedule_buffers(len(exp_rows))
        b = core.batch_params(bt["srcs"], bt["dsts"], chunk, [1] * lanes, segments=bt["segments"])
        _lib.check(lib.flh_stripe_batch_carry(C.byref(b), C.byref(W), C.byref(L), out.table.data_ptr(), out.hdr.data_ptr(), status.data_ptr(), None))
        core.reassemble_batch(b, L, status)
        torch.cuda.synchronize()
        assert int(status.item()) == 0
        got = out.table_numpy()
        for f in ob.DESC_DTYPE.names:
            np.testing.assert_array_equal(got[f], exp_rows[f], err_msg=f)
        for l, off, data in staged:
            np.testing.assert_array_equal(stage[l].cpu().numpy()[off:off + data.size], data, err_msg=f"staging lane {l}")
            np.testing.assert_array_equal(land[l].cpu().numpy()[off:off + data.size], data, err_msg=f"landing lane {l}")
        for i, s in enumerate(bt["sizes"]):
            g = bt["dsts"][i].cpu().numpy()
            np.testing.assert_array_equal(g[:s], bt["srcs_np"][i], err_msg=f"request {i}")
            assert not g[s:].any()


@pytest.mark.parametrize("sets,landing_sets", [(1, 1), (3, 2), (2, 4)])
def test_engine_send_and_receive_halves_equal_the_oracle(fl, sets, landing_sets):
    """A sending engine stripes into its own rotating window sets and carries into landing sets; a second engine -- the
    receiving process's, here in the same process -- delivers out of the landing sets.  A landing set goes back to the
    sender once the receive batch that read it is complete, which is what the plugin's wave counters do."""
    core, torch, _lib = fl
    lib = _lib.load()
    rng = np.random.default_rng(9100 + 10 * sets + landing_sets)
    lanes, chunk, n_batches, cap = 6, 32 << 10, 9, 3 << 20
    tx, rx = C.c_void_p(), C.c_void_p()
    _lib.check(lib.flh_engine_create(0, 0, 100, sets, C.byref(tx)))
    _lib.check(lib.flh_engine_create(0, 65, 100, 8, C.byref(rx)))       # (the receiving side rotates nothing of its own)
    try:
        stage = [[torch.zeros(cap + 64, dtype=torch.uint8, device="cuda") for _ in range(lanes)] for _ in range(sets)]
        land = [[torch.zeros(cap + 64, dtype=torch.uint8, device="cuda") for _ in range(lanes)] for _ in range(landing_sets)]
        W = [core.make_windows([t.data_ptr() for t in ws], [cap] * lanes) for ws in stage]
        L = [core.make_windows([t.data_ptr() for t in ws], [cap] * lanes) for ws in land]
        status = core.new_status()
        batches = [_random_batch(rng, torch, lanes, chunk) for _ in range(n_batches)]
        for bt in batches:
            bt["exp_rows"], bt["staged"] = _expect_batch(bt["segments"], bt["srcs_np"], lanes, chunk)
            bt["out"] = core.new_schedule_buffers(len(bt["exp_rows"]))
        torch.cuda.synchronize()
        sseq, rseq = C.c_uint64(), C.c_uint64()
        sent, received = [], []           # engine numbers of the send and receive batches, by batch
        k_recv = 0
        for k, bt in enumerate(batches):
            if k >= landing_sets:         # the landing set must have been read out by the receive batch that used it last
                while k_recv <= k - landing_sets:
                    _wait(lib, tx, sent[k_recv])
                    rb = batches[k_recv]
                    b = core.batch_params(rb["srcs"], rb["dsts"], chunk, [1] * lanes, segments=rb["segments"])
                    _lib.check(lib.flh_engine_submit_wire(rx, RECV, C.byref(b), C.byref(L[k_recv % landing_sets]), None, None, None, status.data_ptr(),
                                                          C.byref(rseq), None))
                    received.append(rseq.value)
                    k_recv += 1
                _wait(lib, rx, received[k - landing_sets])
            if sets == 1 and sent:
                _wait(lib, tx, sent[-1])
            b = core.batch_params(bt["srcs"], bt["dsts"], chunk, [1] * lanes, segments=bt["segments"])
            _lib.check(lib.flh_engine_submit_wire(tx, SEND, C.byref(b), C.byref(W[k % sets]), C.byref(L[k % landing_sets]), bt["out"].table.data_ptr(),
                                                  bt["out"].hdr.data_ptr(), status.data_ptr(), C.byref(sseq), None))
            assert sseq.value == k + 1
            sent.append(sseq.value)
        while k_recv < n_batches:
            _wait(lib, tx, sent[k_recv])
            rb = batches[k_recv]
            if k_recv >= n_batches - landing_sets:      # the landing sets still hold these batches: compare before they are read out
                for l, off, data in rb["staged"]:
                    np.testing.assert_array_equal(land[k_recv % landing_sets][l].cpu().numpy()[off:off + data.size], data, err_msg=f"batch {k_recv}: landing lane {l}")
            b = core.batch_params(rb["srcs"], rb["dsts"], chunk, [1] * lanes, segments=rb["segments"])
            _lib.check(lib.flh_engine_submit_wire(rx, RECV, C.byref(b), C.byref(L[k_recv % landing_sets]), None, None, None, status.data_ptr(), C.byref(rseq), None))
            received.append(rseq.value)
            k_recv += 1
        _wait(lib, rx, received[-1])
        torch.cuda.synchronize()
        assert int(status.item()) == 0 and lib.flh_engine_error(tx) == 0 and lib.flh_engine_error(rx) == 0
        for k, bt in enumerate(batches):
            got = bt["out"].table_numpy()
            for f in ob.DESC_DTYPE.names:
                np.testing.assert_array_equal(got[f], bt["exp_rows"][f], err_msg=f"batch {k}: {f}")
            for i, s in enumerate(bt["sizes"]):
                g = bt["dsts"][i].cpu().numpy()
                np.testing.assert_array_equal(g[:s], bt["srcs_np"][i], err_msg=f"batch {k} request {i}")
                assert not g[s:].any()
        # the wrong kind of arguments is refused on the host
        b = core.batch_params(batches[0]["srcs"], batches[0]["dsts"], chunk, [1] * lanes, segments=batches[0]["segments"])
        assert lib.flh_engine_submit_wire(tx, SEND, C.byref(b), C.byref(W[0]), None, None, None, status.data_ptr(), C.byref(sseq), None) == -1
        assert lib.flh_engine_submit_wire(rx, RECV, C.byref(b), C.byref(L[0]), C.byref(L[0]), None, None, status.data_ptr(), C.byref(rseq), None) == -1
        assert lib.flh_engine_submit_wire(rx, 0, C.byref(b), C.byref(L[0]), None, None, None, status.data_ptr(), C.byref(rseq), None) == -1
    finally:
        _lib.check(lib.flh_engine_destroy(tx))
        _lib.check(lib.flh_engine_destroy(rx))


def test_landing_windows_used_again_deliver_their_latest_contents(fl):
    """The receiving engine's workers stay resident and read the same landing windows batch after batch; another
    engine's workers (another process's, in the plugin) have written them in between.  What a receive batch delivers
    must be what the latest send batch landed, 40 times over the same buffers, odd sizes among them."""
    core, torch, _lib = fl
    lib = _lib.load()
    rng = np.random.default_rng(517)
    lanes, chunk, cap = 4, 64 << 10, 2 << 20
    tx, rx = C.c_void_p(), C.c_void_p()
    _lib.check(lib.flh_engine_create(0, 0, 5000, 1, C.byref(tx)))
    _lib.check(lib.flh_engine_create(0, 0, 5000, 1, C.byref(rx)))
    try:
        sizes = [3 * chunk, 2 * chunk, 5 * chunk - 777]
        credits = [3, 1, 2, 2]
        srcs = [torch.zeros(s, dtype=torch.uint8, device="cuda") for s in sizes]
        dsts = [torch.zeros(s + 32, dtype=torch.uint8, device="cuda") for s in sizes]
        stage = [torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
        land = [torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
        W = core.make_windows([t.data_ptr() for t in stage], [cap] * lanes)
        L = core.make_windows([t.data_ptr() for t in land], [cap] * lanes)
        status = core.new_status()
        b = core.batch_params(srcs, dsts, chunk, credits)
        side = torch.cuda.Stream()
        sseq, rseq = C.c_uint64(), C.c_uint64()
        for it in range(40):
            fresh = [torch.from_numpy(rng.integers(0, 256, size=s, dtype=np.uint8)).cuda() for s in sizes]
            with torch.cuda.stream(side):           # a kernel on another stream writes the sources the engine has read before
                for s_, f_ in zip(srcs, fresh):
                    s_.copy_(f_)
            side.synchronize()
            _lib.check(lib.flh_engine_submit_wire(tx, SEND, C.byref(b), C.byref(W), C.byref(L), None, None, status.data_ptr(), C.byref(sseq), None))
            _wait(lib, tx, sseq.value)
            _lib.check(lib.flh_engine_submit_wire(rx, RECV, C.byref(b), C.byref(L), None, None, None, status.data_ptr(), C.byref(rseq), None))
            _wait(lib, rx, rseq.value)
            with torch.cuda.stream(side):           # compared by a kernel that starts once the batch is reported complete
                same = all(bool(torch.equal(d_[:s], f_)) for d_, f_, s in zip(dsts, fresh, sizes))
            assert same, f"iteration {it}: a receive batch delivered stale bytes"
        assert int(status.item()) == 0
    finally:
        _lib.check(lib.flh_engine_destroy(tx))
        _lib.check(lib.flh_engine_destroy(rx))


def test_the_engine_leaves_when_its_time_is_up_and_work_goes_on(fl):
    """A resident kernel holds its hardware queue.  With a bound on its residency the engine leaves between two batches
    although batches keep coming; the submit that finds it down -- or flh_engine_poke, when nothing further is submitted
    -- starts the next one, and no batch is lost or executed twice."""
    core, torch, _lib = fl
    lib = _lib.load()
    rng = np.random.default_rng(233)
    lanes, chunk, cap, sets = 4, 64 << 10, 2 << 20, 3
    eng = C.c_void_p()
    _lib.check(lib.flh_engine_create(0, 0, 100000, sets, C.byref(eng)))      # it would idle out only after 100 ms
    _lib.check(lib.flh_engine_set_resident(eng, 300))                        # ... but leaves after 300 us
    try:
        wins = [[torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)] for _ in range(sets)]
        W = [core.make_windows([t.data_ptr() for t in ws], [cap] * lanes) for ws in wins]
        status = core.new_status()
        n = 6 * chunk
        src_np = rng.integers(0, 256, size=n, dtype=np.uint8)
        src = _dev(torch, src_np)
        n_batches = 60
        dsts = [torch.zeros(n, dtype=torch.uint8, device="cuda") for _ in range(n_batches)]
        torch.cuda.synchronize()
        seq = C.c_uint64()
        t0 = time.time()
        for k in range(n_batches):
            b = core.batch_params([src], [dsts[k]], chunk, [2, 1, 1, 3], epoch_bytes=k * n)
            _lib.check(lib.flh_engine_submit(eng, C.byref(b), C.byref(W[k % sets]), None, None, status.data_ptr(), C.byref(seq), None))
            if k >= sets - 1:
                _wait(lib, eng, seq.value - (sets - 1))
            if k == 20:
                time.sleep(0.002)          # the engine's time runs out with nothing submitted: it leaves with batches done, the next submit starts it
        _wait(lib, eng, seq.value)
        elapsed = time.time() - t0
        launches = int(lib.flh_engine_launches(eng))
        assert launches >= 2, f"{launches} engine launches in {elapsed * 1e3:.1f} ms with a 300 us bound"
        assert lib.flh_engine_error(eng) == 0 and int(status.item()) == 0
        for k in range(n_batches):
            np.testing.assert_array_equal(dsts[k].cpu().numpy(), src_np, err_msg=f"batch {k}")
        # nothing outstanding: nothing to start
        time.sleep(0.001)
        assert lib.flh_engine_needs_start(eng) == 0 and lib.flh_engine_poke(eng) == 0
        assert int(lib.flh_engine_launches(eng)) == launches
    finally:
        _lib.check(lib.flh_engine_destroy(eng))


def test_a_submit_that_fails_is_final(fl):
    """When the resident kernel cannot be started, flh_engine_submit returns the error with the batch taken back out of
    the ring: the caller carries it some other way, and the engine, once it can be started again, must not execute it as
    well -- its buffers have been given away by then."""
    core, torch, _lib = fl
    lib = _lib.load()
    lanes, chunk, cap = 4, 64 << 10, 2 << 20
    eng = C.c_void_p()
    _lib.check(lib.flh_engine_create(0, 0, 200, 2, C.byref(eng)))
    try:
        wins = [torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
        W = core.make_windows([t.data_ptr() for t in wins], [cap] * lanes)
        status = core.new_status()
        n = 4 * chunk
        src_a = torch.full((n,), 0xAA, dtype=torch.uint8, device="cuda")
        src_b = torch.full((n,), 0xBB, dtype=torch.uint8, device="cuda")
        dst_a = torch.zeros(n, dtype=torch.uint8, device="cuda")
        dst_b = torch.zeros(n, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        seq = C.c_uint64()
        _lib.check(lib.flh_tune(b"engine_fail_start", 1))
        try:
            ba = core.batch_params([src_a], [dst_a], chunk, [1] * lanes)
            assert lib.flh_engine_submit(eng, C.byref(ba), C.byref(W), None, None, status.data_ptr(), C.byref(seq), None) == -2     # FLH_E_HIP
            assert b"engine launch failed" in lib.flh_last_error()
        finally:
            _lib.check(lib.flh_tune(b"engine_fail_start", 0))
        assert int(lib.flh_engine_completed(eng)) == 0 and int(lib.flh_engine_launches(eng)) == 0 and lib.flh_engine_needs_start(eng) == 0
        bb = core.batch_params([src_b], [dst_b], chunk, [1] * lanes)
        _lib.check(lib.flh_engine_submit(eng, C.byref(bb), C.byref(W), None, None, status.data_ptr(), C.byref(seq), None))
        assert seq.value == 1                        # the number the failed batch had been given
        _wait(lib, eng, 1)
        time.sleep(0.005)
        torch.cuda.synchronize()
        assert int(lib.flh_engine_completed(eng)) == 1
        assert (dst_b.cpu().numpy() == 0xBB).all()
        assert not dst_a.cpu().numpy().any(), "the batch whose submit failed was executed after all"
        assert lib.flh_engine_error(eng) == 0
    finally:
        _lib.check(lib.flh_engine_destroy(eng))


def test_test_hooks_are_refused_without_their_switch(fl, monkeypatch):
    core, torch, _lib = fl
    lib = _lib.load()
    monkeypatch.delenv("NCCL_FUSELINK_TEST_HOOKS", raising=False)
    for key in (b"engine_fail_start", b"engine_inject_fault", b"engine_wait_us"):
        assert lib.flh_tune(key, 1) == -6
    monkeypatch.setenv("NCCL_FUSELINK_TEST_HOOKS", "1")
    assert lib.flh_tune(b"engine_fail_start", 0) == 0


# ---- stage + deliver in one launch: the sender writes the receive buffer itself ---------------------------------------

@pytest.mark.parametrize("nbytes,chunk,lanes,epoch_chunks,src_skew,win_skew,dst_skew", [
    ((4 << 20) + 4096 + 3, 256 << 10, 8, 0, 0, 0, 0), (64 << 20, 256 << 10, 8, 5, 0, 0, 0), (7 * (96 << 10) + 1, 96 << 10, 3, 2, 0, 0, 0),
    ((3 << 20) + 77, 128 << 10, 4, 1, 5, 5, 5),   # source, windows and receive buffer equally misaligned: vectors with byte edges
    ((3 << 20) + 77, 128 << 10, 4, 1, 0, 0, 9),   # the receive buffer misaligned against source and windows: two copies from the source
    ((1 << 20) + 13, 100 * 128, 5, 3, 3, 0, 3),   # the windows misaligned against source and receive buffer
    (5 * (256 << 10) + 6 * 32768 + 16392, 256 << 10, 5, 0, 0, 0, 0),   # a last tile of 16 KiB and a few bytes: the four-vector path
    (3 * (64 << 10) + 16384, 64 << 10, 2, 1, 0, 0, 0),
    (300 << 20, 1 << 20, 16, 0, 0, 0, 0)])        # past 256 MiB: destination order, streaming loads and stores
def test_a_launch_that_stages_and_delivers_equals_the_launch_pair(fl, nbytes, chunk, lanes, epoch_chunks, src_skew, win_skew, dst_skew):
    """flh_stage_deliver_uniform: table, header and windows are flh_stripe_uniform's, the receive buffer
    flh_reassemble_uniform's -- the oracle's -- and the bytes around the receive buffer stay untouched."""
    core, torch, _lib = fl
    lib = _lib.load()
    rng = np.random.default_rng(nbytes % 9973 + lanes + dst_skew)
    credits = rng.integers(1, 9, size=lanes).astype(np.uint32)
    epoch = epoch_chunks * chunk
    src_np = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=nbytes, chunk_bytes=chunk,
                                         mode=ob.SCHED_RESET_OFFSETS, state=_state(epoch))
    lane_bytes = [int(x) for x in exp_h["lane_bytes"][:lanes]]
    src_buf = torch.zeros(nbytes + 64, dtype=torch.uint8, device="cuda")
    src = src_buf[src_skew:src_skew + nbytes]
    src.copy_(torch.from_numpy(src_np))
    dst_buf = torch.full((nbytes + 128,), 0xEE, dtype=torch.uint8, device="cuda")
    dst = dst_buf[32 + dst_skew:32 + dst_skew + nbytes]
    stage_buf = [torch.zeros(max(b, 1) + 64, dtype=torch.uint8, device="cuda") for b in lane_bytes]
    stage = [t[win_skew:] for t in stage_buf]
    W = core.make_windows([t.data_ptr() for t in stage], lane_bytes)
    status = core.new_status()
    out = core.new_schedule_buffers(len(exp_t))
    u = core.uniform_params(nbytes, chunk, credits.tolist(), epoch_bytes=epoch)
    done = torch.zeros(64, dtype=torch.int32).pin_memory()
    count = torch.zeros(64, dtype=torch.int32, device="cuda")
    if nbytes < (8 << 20):
        u.d_done_word, u.d_done_count, u.done_value = done.data_ptr(), count.data_ptr(), 43
    core.stage_deliver_uniform(src, dst, W, u, status, out=out)
    if nbytes < (8 << 20):
        deadline = time.time() + 10
        while int(done[0]) != 43:
            assert time.time() < deadline, "the completion word never came"
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and int(count[0].item()) == 0
    got = out.table_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got[f], exp_t[f], err_msg=f)
    np.testing.assert_array_equal(out.hdr_numpy()["lane_bytes"][:lanes], exp_h["lane_bytes"][:lanes])
    if nbytes <= (64 << 20):
        exp_w = ob.cpu_stripe(src_np, exp_t, lane_bytes)
        for l in range(lanes):
            np.testing.assert_array_equal(stage[l].cpu().numpy()[:lane_bytes[l]], exp_w[l][:lane_bytes[l]], err_msg=f"staging window {l}")
            assert not stage[l].cpu().numpy()[lane_bytes[l]:].any()
    else:   # the windows, taken apart again by the reassembly launch, give the message back
        back = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        core.reassemble_uniform(back, W, u, status)
        torch.cuda.synchronize()
        assert torch.equal(back, src)
    back = dst_buf.cpu().numpy()
    lo = 32 + dst_skew
    np.testing.assert_array_equal(back[lo:lo + nbytes], src_np)
    assert (back[:lo] == 0xEE).all() and (back[lo + nbytes:] == 0xEE).all()


def test_a_delivery_that_would_leave_the_receive_buffer_is_refused(fl):
    core, torch, _lib = fl
    lib = _lib.load()
    lanes, chunk, nbytes = 2, 64 << 10, 8 * (64 << 10)
    src = torch.ones(nbytes, dtype=torch.uint8, device="cuda")
    dst = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    stage = [torch.zeros(4 * chunk, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
    W = core.make_windows([t.data_ptr() for t in stage], [4 * chunk] * lanes)
    status = core.new_status()
    u = core.uniform_params(nbytes, chunk, [1, 1])
    # the receive buffer is said to end one chunk early: the last chunk goes nowhere, not even into its window
    _lib.check(lib.flh_stage_deliver_uniform(src.data_ptr(), nbytes, dst.data_ptr(), nbytes - chunk, C.byref(W), C.byref(u), None, None, status.data_ptr(), None))
    torch.cuda.synchronize()
    assert int(status.item()) == -5                                                   # FLH_E_RANGE
    d = dst.cpu().numpy()
    assert d[:nbytes - chunk].all() and not d[nbytes - chunk:].any()
    assert not stage[1].cpu().numpy()[3 * chunk:].any() and stage[0].cpu().numpy().all()
    assert lib.flh_stage_deliver_uniform(src.data_ptr(), nbytes, None, nbytes, C.byref(W), C.byref(u), None, None, status.data_ptr(), None) == -1


def test_a_batch_launch_that_stages_and_delivers_equals_the_batch_pair(fl):
    core, torch, _lib = fl
    lib = _lib.load()
    rng = np.random.default_rng(812)
    lanes, chunk, cap = 5, 32 << 10, 3 << 20
    for _ in range(6):
        bt = _random_batch(rng, torch, lanes, chunk)
        stage = [torch.zeros(cap, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
        W = core.make_windows([t.data_ptr() for t in stage], [cap] * lanes)
        status = core.new_status()
        exp_rows, staged = _expect_batch(bt["segments"], bt["srcs_np"], lanes, chunk)
        out = core.new_schedule_buffers(len(exp_rows))
        b = core.batch_params(bt["srcs"], bt["dsts"], chunk, [1] * lanes, segments=bt["segments"])
        _lib.check(lib.flh_stage_deliver_batch(C.byref(b), C.byref(W), out.table.data_ptr(), out.hdr.data_ptr(), status.data_ptr(), None))
        torch.cuda.synchronize()
        assert int(status.item()) == 0
        got = out.table_numpy()
        for f in ob.DESC_DTYPE.names:
            np.testing.assert_array_equal(got[f], exp_rows[f], err_msg=f)
        for l, off, data in staged:
            np.testing.assert_array_equal(stage[l].cpu().numpy()[off:off + data.size], data, err_msg=f"staging lane {l}")
        for i, s in enumerate(bt["sizes"]):
            g = bt["dsts"][i].cpu().numpy()
            np.testing.assert_array_equal(g[:s], bt["srcs_np"][i], err_msg=f"request {i}")
            assert not g[s:].any()


_LAST = [1, 7, 15, 16, 17, 31, 32, 255, 256, 4095, 4096, 4097, 8191, 8192, 12288, 16383, 16384, 16385, 16392, 16399, 16400, 20480, 24576, 28672,
         32752, 32760, 32767]


@pytest.mark.parametrize("skew", [0, 4])
def test_every_size_class_of_a_last_tile_reaches_both_destinations(fl, skew):
    """The copy with two destinations takes different paths by the number of 16-byte vectors in a tile (whole tiles
    unrolled, anything else in a predicated loop, bytes at either edge).  Messages of a chunk, a tile and a last tile of
    every size class -- around every power of two, sixteen kilobytes and a few bytes, a tile less a few -- go through the
    launch that stages and delivers, the launch that stages and carries, and the engine's two kinds of batch that do
    the same at system scope (one-tile and, with the share limit at 0, two-tile shares); source, windows and
    destinations share a misalignment of `skew` bytes so that the vector path is the one taken.  Windows, landing
    windows and destinations must hold exactly the message, and nothing beside it."""
    core, torch, _lib = fl
    lib = _lib.load()
    lib.flh_tune.argtypes = [C.c_char_p, C.c_int64]
    lanes, chunk = 2, 64 << 10
    credits = [1, 1]
    rng = np.random.default_rng(77 + skew)
    cap = 4 * chunk
    status = core.new_status()

    def buffers(n, fill):
        raw = [torch.full((n + 64,), fill, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
        return raw, [t[skew:skew + n] for t in raw]

    def check(name, last, src_np, exp_w, lane_bytes, stage, land, dst_raw, fill):
        for l in range(lanes):
            np.testing.assert_array_equal(stage[l].cpu().numpy()[:lane_bytes[l]], exp_w[l][:lane_bytes[l]], err_msg=f"{name}, last {last}: staging window {l}")
            assert (stage[l].cpu().numpy()[lane_bytes[l]:] == 0).all(), f"{name}, last {last}: staging window {l} written beyond its bytes"
            if land is not None:
                np.testing.assert_array_equal(land[l].cpu().numpy()[:lane_bytes[l]], exp_w[l][:lane_bytes[l]], err_msg=f"{name}, last {last}: landing window {l}")
                assert (land[l].cpu().numpy()[lane_bytes[l]:] == 0).all(), f"{name}, last {last}: landing window {l} written beyond its bytes"
        if dst_raw is not None:
            back = dst_raw.cpu().numpy()
            np.testing.assert_array_equal(back[32 + skew:32 + skew + src_np.size], src_np, err_msg=f"{name}, last {last}: destination")
            assert (back[:32 + skew] == fill).all() and (back[32 + skew + src_np.size:] == fill).all(), f"{name}, last {last}: bytes around the destination"

    for share_limit in (-1, 0):
        _lib.check(lib.flh_tune(b"lane_share1_tiles", share_limit))
        eng = C.c_void_p()
        _lib.check(lib.flh_engine_create(0, 0, 200, 1, C.byref(eng)))
        try:
            for last in _LAST:
                nbytes = chunk + 32768 + last
                src_np = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
                src_raw = torch.zeros(nbytes + 64, dtype=torch.uint8, device="cuda")
                src = src_raw[skew:skew + nbytes]
                src.copy_(torch.from_numpy(src_np))
                exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=np.asarray(credits, dtype=np.uint32), quantum=chunk, total_bytes=nbytes,
                                                     chunk_bytes=chunk, mode=ob.SCHED_RESET_OFFSETS, state=_state(0))
                lane_bytes = [int(x) for x in exp_h["lane_bytes"][:lanes]]
                exp_w = ob.cpu_stripe(src_np, exp_t, lane_bytes)
                u = core.uniform_params(nbytes, chunk, credits)
                for name in (("deliver", "carry") if share_limit == -1 else ()) + ("engine loop", "engine send"):
                    _, stage = buffers(cap, 0)
                    _, land = buffers(cap, 0)
                    W = core.make_windows([t.data_ptr() for t in stage], [cap] * lanes)
                    L = core.make_windows([t.data_ptr() for t in land], [cap] * lanes)
                    dst_raw = torch.full((nbytes + 128,), 0xEE, dtype=torch.uint8, device="cuda")
                    dst = dst_raw[32 + skew:32 + skew + nbytes]
                    torch.cuda.synchronize()
                    if name == "deliver":
                        core.stage_deliver_uniform(src, dst, W, u, status)
                    elif name == "carry":
                        core.stripe_uniform_carry(src, W, L, u, status)
                    else:
                        b = core.batch_params([src], [dst], chunk, credits)
                        seq = C.c_uint64()
                        if name == "engine loop":
                            _lib.check(lib.flh_engine_submit(eng, C.byref(b), C.byref(W), None, None, status.data_ptr(), C.byref(seq), None))
                        else:
                            _lib.check(lib.flh_engine_submit_wire(eng, SEND, C.byref(b), C.byref(W), C.byref(L), None, None, status.data_ptr(), C.byref(seq), None))
                        _wait(lib, eng, seq.value)
                    torch.cuda.synchronize()
                    assert int(status.item()) == 0
                    check(name, last, src_np, exp_w, lane_bytes, stage, land if name in ("carry", "engine send") else None,
                          dst_raw if name in ("deliver", "engine loop") else None, 0xEE)
        finally:
            _lib.check(lib.flh_tune(b"lane_share1_tiles", -1))
            _lib.check(lib.flh_engine_destroy(eng))


@pytest.mark.parametrize("block", range(int(__import__("os").environ.get("FUSELINK_TWO_DEST_BLOCKS", "2"))))
def test_random_messages_through_the_two_destination_paths(fl, block):
    """Seeded random messages -- length, chunk size (any multiple of 128), lanes, credit row, place in the credit epoch, and
    the misalignments of source, windows and destination against each other -- through the launch that stages and
    delivers, the launch that stages and carries, and the engine's loop and send batches: windows, landing windows and
    destination must be the oracle's, byte for byte, and the bytes beside them untouched.  Forty cases per block."""
    core, torch, _lib = fl
    lib = _lib.load()
    rng = np.random.default_rng(31000 + block)
    status = core.new_status()
    eng = C.c_void_p()
    _lib.check(lib.flh_engine_create(0, 0, 200, 1, C.byref(eng)))
    try:
        for case in range(40):
            lanes = int(rng.integers(1, 9))
            chunk = int(rng.choice([128, 4096, 12800, 32768, 65536, 98304, 262144]))
            n_chunks = int(rng.integers(1, 24))
            nbytes = max(1, (n_chunks - 1) * chunk + int(rng.integers(1, chunk + 1)))
            credits = rng.integers(0, 5, size=lanes).astype(np.uint32)
            epoch = int(rng.integers(0, 20)) * chunk
            same = rng.random() < 0.6                       # mostly the vector path: every address misaligned alike
            s0 = int(rng.integers(0, 16))
            skews = (s0, s0, s0) if same else tuple(int(x) for x in rng.integers(0, 16, size=3))
            src_np = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
            exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=nbytes, chunk_bytes=chunk,
                                                 mode=ob.SCHED_RESET_OFFSETS, state=_state(epoch))
            lane_bytes = [int(x) for x in exp_h["lane_bytes"][:lanes]]
            exp_w = ob.cpu_stripe(src_np, exp_t, lane_bytes)
            src_raw = torch.zeros(nbytes + 64, dtype=torch.uint8, device="cuda")
            src = src_raw[skews[0]:skews[0] + nbytes]
            src.copy_(torch.from_numpy(src_np))
            u = core.uniform_params(nbytes, chunk, credits.tolist(), epoch_bytes=epoch)
            for name in ("deliver", "carry", "engine loop", "engine send"):
                if name.startswith("engine") and (n_chunks > 500 or chunk % 128):
                    continue
                tag = f"block {block} case {case} {name}: {nbytes} bytes, chunk {chunk}, lanes {lanes}, credits {credits.tolist()}, epoch {epoch}, skews {skews}"
                stage_raw = [torch.full((b + 64,), 0x5A, dtype=torch.uint8, device="cuda") for b in lane_bytes]
                land_raw = [torch.full((b + 64,), 0x5A, dtype=torch.uint8, device="cuda") for b in lane_bytes]
                W = core.make_windows([t.data_ptr() + skews[1] for t in stage_raw], lane_bytes)
                L = core.make_windows([t.data_ptr() + skews[1] for t in land_raw], lane_bytes)
                dst_raw = torch.full((nbytes + 128,), 0xEE, dtype=torch.uint8, device="cuda")
                dst = dst_raw[32 + skews[2]:32 + skews[2] + nbytes]
                torch.cuda.synchronize()
                if name == "deliver":
                    core.stage_deliver_uniform(src, dst, W, u, status)
                elif name == "carry":
                    core.stripe_uniform_carry(src, W, L, u, status)
                else:
                    b = core.batch_params([src], [dst], chunk, credits.tolist(), epoch_bytes=epoch)
                    seq = C.c_uint64()
                    if name == "engine loop":
                        _lib.check(lib.flh_engine_submit(eng, C.byref(b), C.byref(W), None, None, status.data_ptr(), C.byref(seq), None))
                    else:
                        _lib.check(lib.flh_engine_submit_wire(eng, SEND, C.byref(b), C.byref(W), C.byref(L), None, None, status.data_ptr(), C.byref(seq), None))
                    _wait(lib, eng, seq.value)
                torch.cuda.synchronize()
                assert int(status.item()) == 0, tag
                for l in range(lanes):
                    for kind, raw in (("staging", stage_raw), ("landing", land_raw)):
                        if kind == "landing" and name not in ("carry", "engine send"):
                            continue
                        g = raw[l].cpu().numpy()
                        np.testing.assert_array_equal(g[skews[1]:skews[1] + lane_bytes[l]], exp_w[l][:lane_bytes[l]], err_msg=f"{tag}: {kind} window {l}")
                        assert (g[:skews[1]] == 0x5A).all() and (g[skews[1] + lane_bytes[l]:] == 0x5A).all(), f"{tag}: bytes beside {kind} window {l}"
                if name in ("deliver", "engine loop"):
                    back = dst_raw.cpu().numpy()
                    lo = 32 + skews[2]
                    np.testing.assert_array_equal(back[lo:lo + nbytes], src_np, err_msg=f"{tag}: destination")
                    assert (back[:lo] == 0xEE).all() and (back[lo + nbytes:] == 0xEE).all(), f"{tag}: bytes beside the destination"
    finally:
        _lib.check(lib.flh_engine_destroy(eng))
