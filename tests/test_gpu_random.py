"""Randomised parity: scheduler and copy entry points against the oracle on seeded random shapes -- lanes,
credit rows (empty rows, sums past 16 bits), epochs, tiles, carried state, every mode bit, ragged and
misaligned buffers, destination order, batches.  Each case is small; the point is the breadth of shapes."""
import numpy as np
import pytest

from tests import oracle_binding as ob

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fl():
    import torch

    from fuselink_amd import core
    core.init(0)
    return core, torch


def _dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _same(got, exp, what):
    for f in ob.DESC_DTYPE.names:
        if not np.array_equal(got[f], exp[f]):
            i = int(np.nonzero(got[f] != exp[f])[0][0])
            raise AssertionError(f"{what}: field {f} differs at row {i}: got {got[f][i]} exp {exp[f][i]}")


def _schedule_case(core, torch, seed):
    dev = lambda a: _dev(torch, a)  # noqa: E731
    same = _same
    rng = np.random.default_rng(seed)
    lanes = int(rng.integers(1, 17))
    rows = int(rng.integers(1, 40))
    hi = int(rng.choice([2, 9, 1000, 2**20]))
    credits = rng.integers(0, hi, size=(rows, lanes)).astype(np.uint32)
    if rng.random() < 0.3:
        credits[rng.integers(0, rows)] = 0
    epoch_len = int(rng.choice([0, 1, 2, 7, 64, 1000]))
    tile = int(rng.choice([128, 4096, 32768, 3*128]))
    mode = int(rng.choice([0, 1, 4, 5, 2]))
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["chunk_index"] = int(rng.integers(0, 5000))
    st["epoch_bytes"] = int(rng.integers(0, 1 << int(rng.choice([24, 41]))))      # carried prefixes past 32 bits too
    st["lane_off"][:lanes] = rng.integers(0, 1 << int(rng.choice([30, 45])), size=lanes)
    kind = int(rng.integers(0, 3))
    what = f"seed {seed} kind {kind} lanes {lanes} rows {rows} E {epoch_len} tile {tile} mode {mode}"
    if kind == 0:   # variable sizes, scan kernel
        n = int(rng.choice([1, 5, 64, 65, 300, 513, 1100, 2049, 5000]))
        quantum = int(rng.choice([1, 4096, 65536, 100000, 1 << 20]))
        sizes = rng.integers(0, int(rng.choice([2, 5000, 300000, 1 << 22])), size=n).astype(np.uint32)
        exp_t, exp_h, exp_s = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=quantum, sizes=sizes, epoch_len=epoch_len, tile_bytes=tile, mode=mode, state=st)
        d_state = dev(np.array([st], dtype=ob.STATE_DTYPE).view(np.uint8))
        sched = core.schedule(n_lanes=lanes, credits=dev(credits.view(np.int32)), quantum=quantum, sizes=dev(sizes.view(np.int32)), epoch_len=epoch_len, tile_bytes=tile, mode=mode, state=d_state)
    else:           # uniform split: closed form (kind 1) or forced scan (kind 2)
        chunk = int(rng.choice([128, 4096, 65536, 100*128]))
        n = int(rng.choice([1, 2, 255, 256, 257, 1000, 3000, 9000]))
        total = n*chunk - int(rng.integers(0, chunk))
        rows_c = credits[:32] if kind == 1 else credits
        exp_t, exp_h, exp_s = ob.credit_schedule(n_lanes=lanes, credits=rows_c, quantum=chunk, total_bytes=total, chunk_bytes=chunk, epoch_len=epoch_len, tile_bytes=tile, mode=mode, state=st)
        d_state = dev(np.array([st], dtype=ob.STATE_DTYPE).view(np.uint8))
        core.tune("sched_uniform_fast", 1 if kind == 1 else 0)
        by_lane = kind == 1 and rng.random() < 0.5
        sched = core.schedule(n_lanes=lanes, credits=dev(rows_c.view(np.int32)), quantum=chunk, total_bytes=total, chunk_bytes=chunk, epoch_len=epoch_len, tile_bytes=tile, mode=mode, state=d_state, by_lane=by_lane)
        core.tune("sched_uniform_fast", 1)
        if by_lane:
            torch.cuda.synchronize()
            same(sched.table_by_lane_numpy(), ob.table_by_lane(exp_t, lanes, (chunk + tile - 1)//tile), what + " by-lane")
    torch.cuda.synchronize()
    same(sched.table_numpy(), exp_t, what)
    gh = sched.hdr_numpy()
    for f in ("total_bytes", "total_tiles", "n_chunks", "flags", "lane_bytes", "lane_chunks"):
        assert np.array_equal(gh[f], exp_h[f]), (what, f, gh[f], exp_h[f])
    gs = core.state_numpy(d_state)
    for f in ob.STATE_DTYPE.names:
        assert np.array_equal(gs[f], exp_s[f]), (what, "state", f, gs[f], exp_s[f])


@pytest.mark.parametrize("block", range(8))
def test_random_schedules_match_the_oracle(fl, block):
    core, torch = fl
    try:
        for seed in range(block * 60, block * 60 + 60):
            _schedule_case(core, torch, 900_000 + seed)
    finally:
        core.tune("sched_uniform_fast", 1)


def _copy_case(core, torch, seed, status):
    dev = lambda a: _dev(torch, a)  # noqa: E731
    rng = np.random.default_rng(seed)
    lanes = int(rng.integers(1, 17))
    credits = rng.integers(0, int(rng.choice([2, 9, 300])), size=lanes).astype(np.uint32)
    tile = int(rng.choice([128, 4096, 32768, 3*128]))
    kind = int(rng.integers(0, 4))
    what = f"seed {seed} kind {kind} lanes {lanes} tile {tile}"
    if kind == 0:     # variable sizes, explicit offsets with gaps and odd alignment, generic kernel
        n = int(rng.integers(1, 40))
        sizes = rng.integers(0, int(rng.choice([50, 5000, 70000])), size=n).astype(np.uint32)
        gaps = rng.integers(0, 40, size=n)
        offs = np.concatenate([[int(rng.integers(0, 64))], (sizes[:-1] + gaps[:-1])]).cumsum().astype(np.uint64)
        total = int(offs[-1] + sizes[-1]) + 8
        quantum = int(rng.choice([1, 4096, 65536]))
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=quantum, sizes=sizes, src_off=offs, tile_bytes=tile)
        sched = core.schedule(n_lanes=lanes, credits=credits.tolist(), quantum=quantum, sizes=dev(sizes.view(np.int32)), src_off=dev(offs.view(np.int64)), tile_bytes=tile)
        src_np = rng.integers(0, 256, size=total, dtype=np.uint8)
        caps = [int(b) for b in exp_h["lane_bytes"][:lanes]]
        pad = [int(rng.integers(0, 16)) for _ in caps]      # misaligned window bases
        wins = [torch.zeros(c + 64, dtype=torch.uint8, device="cuda") for c in caps]
        w = core.make_windows([t.data_ptr() + p for t, p in zip(wins, pad)], caps)
        src = dev(src_np)
        dst = torch.zeros_like(src)
        core.stripe(src, w, sched, status)
        core.reassemble(dst, w, sched, status)
        torch.cuda.synchronize()
        exp_w = ob.cpu_stripe(src_np, exp_t, caps)
        for l in range(lanes):
            got = wins[l].cpu().numpy()
            assert np.array_equal(got[pad[l]: pad[l] + caps[l]], exp_w[l][: caps[l]]), (what, "window", l)
            assert not got[:pad[l]].any() and not got[pad[l] + caps[l]:].any(), (what, "guard", l)
        exp_dst = np.zeros_like(src_np)
        for r in exp_t:
            exp_dst[int(r["src_off"]): int(r["src_off"]) + int(r["len"])] = src_np[int(r["src_off"]): int(r["src_off"]) + int(r["len"])]
        assert np.array_equal(dst.cpu().numpy(), exp_dst), (what, "dst")
    else:
        chunk = int(rng.choice([128, 4096, 65536, 100*128, 3*128]))
        n = int(rng.integers(1, 60))
        total = n*chunk - int(rng.integers(0, chunk))
        epoch_bytes = int(rng.integers(0, 30))*chunk
        st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
        st["epoch_bytes"] = epoch_bytes
        base = int(rng.integers(0, 5))*int(rng.choice([1, 16, 4096])) if kind != 3 else 0
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk, tile_bytes=tile, mode=1, state=st, src_base=base)
        caps = [int(b) for b in exp_h["lane_bytes"][:lanes]]
        wins = [torch.zeros(c + 64, dtype=torch.uint8, device="cuda") for c in caps]
        w = core.make_windows([t.data_ptr() for t in wins], caps)
        src_np = rng.integers(0, 256, size=base + total, dtype=np.uint8)
        exp_w = ob.cpu_stripe(src_np, exp_t, caps) if kind != 3 else None
        if kind == 1:   # fused, chunk or destination order
            core.tune("stripe_dest_order", int(rng.integers(0, 2)))
            u = core.uniform_params(total, chunk, credits.tolist(), src_base=base, epoch_bytes=epoch_bytes, tile_bytes=tile)
            out = core.new_schedule_buffers(n, tile)
            src = dev(src_np)
            dst = torch.zeros_like(src)
            core.stripe_uniform(src, w, u, status, out=out)
            core.reassemble_uniform(dst, w, u, status)
            torch.cuda.synchronize()
            core.tune("stripe_dest_order", -1)
            assert out.table_numpy().tobytes() == exp_t.tobytes(), (what, "table")
            assert np.array_equal(dst.cpu().numpy()[base:], src_np[base:]) and not dst.cpu().numpy()[:base].any(), (what, "dst")
        elif kind == 2:  # scheduler kernel + table-driven copies, with and without the host hint, rows by lane or by chunk
            by_lane = bool(rng.integers(0, 2))
            d_state = dev(np.array([st], dtype=ob.STATE_DTYPE).view(np.uint8))
            sched = core.schedule(n_lanes=lanes, credits=credits.tolist(), quantum=chunk, total_bytes=total, chunk_bytes=chunk, tile_bytes=tile, mode=1, state=d_state, src_base=base, by_lane=by_lane)
            hint = core.uniform_hint(total, chunk, tile) if rng.integers(0, 2) else None
            src = dev(src_np)
            dst = torch.zeros_like(src)
            core.stripe(src, w, sched, status, hint=hint, by_lane=by_lane)
            core.reassemble(dst, w, sched, status, hint=hint)
            torch.cuda.synchronize()
            assert np.array_equal(dst.cpu().numpy()[base:], src_np[base:]), (what, "dst")
        else:            # batch of requests
            n_req = int(rng.integers(1, 9))
            cuts = sorted(rng.choice(np.arange(1, n), size=min(n_req - 1, n - 1), replace=False).tolist()) if n > 1 else []
            bounds = [0] + [c*chunk for c in cuts] + [total]
            sizes = [b - a for a, b in zip(bounds[:-1], bounds[1:])]
            srcs_np = [src_np[a:b] for a, b in zip(bounds[:-1], bounds[1:])]
            srcs = [dev(x) for x in srcs_np]
            dsts = [torch.zeros(s + 16, dtype=torch.uint8, device="cuda") for s in sizes]
            b = core.batch_params(srcs, dsts, chunk, credits.tolist(), epoch_bytes=epoch_bytes, tile_bytes=tile)
            out = core.new_schedule_buffers(n, tile)
            core.stripe_batch(b, w, status, out=out)
            core.reassemble_batch(b, w, status)
            torch.cuda.synchronize()
            assert out.table_numpy().tobytes() == exp_t.tobytes(), (what, "table")
            exp_w = ob.cpu_stripe(src_np, exp_t, caps)
            for q in range(len(sizes)):
                g = dsts[q].cpu().numpy()
                assert np.array_equal(g[:sizes[q]], srcs_np[q]) and not g[sizes[q]:].any(), (what, "dst", q)
        for l in range(lanes):
            got = wins[l].cpu().numpy()
            assert np.array_equal(got[: caps[l]], exp_w[l][: caps[l]]), (what, "window", l)
            assert not got[caps[l]:].any(), (what, "guard", l)
    assert int(status.item()) == 0, what


@pytest.mark.parametrize("block", range(8))
def test_random_copies_match_the_oracle(fl, block):
    core, torch = fl
    status = core.new_status()
    try:
        for seed in range(block * 40, block * 40 + 40):
            _copy_case(core, torch, 800_000 + seed, status)
    finally:
        core.tune("stripe_dest_order", -1)
