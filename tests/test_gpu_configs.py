"""The benchmark configurations and the staging-window layer on a real MI355X, through the C ABI:
golden schedule vectors, HIP-VMM pool / window / region behaviour (first-fit slots, exhaustion,
refcounts, pointer translation), the expert-parallel send set, the paged KV-cache gather and the
1 GiB stress shape.  Bit-exact against the CPU oracle; at full size through round trips."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from tests import oracle_binding as ob

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat_vectors.json")))
MB = 1 << 20


@pytest.fixture(scope="module")
def fl():
    import torch
    from fuselink_amd import core
    core.init(0)
    return core, torch


def _dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("v", KAT["schedule"], ids=[v["name"][:40] for v in KAT["schedule"]])
def test_scheduler_kernel_against_hand_vectors(fl, v):
    core, torch = fl
    credits = _dev(torch, np.asarray(v["credits"], dtype=np.int32))
    kw = dict(n_lanes=v["n_lanes"], credits=credits, quantum=v["quantum"], epoch_len=v["epoch_len"], tile_bytes=v["tile_bytes"])
    if "sizes" in v:
        kw["sizes"] = _dev(torch, np.asarray(v["sizes"], dtype=np.int32))
    else:
        kw["total_bytes"], kw["chunk_bytes"] = v["total_bytes"], v["chunk_bytes"]
    sched = core.schedule(**kw)
    torch.cuda.synchronize()
    t, h = sched.table_numpy(), sched.hdr_numpy()
    for f in ("lane", "win_off", "src_off", "tile_base", "epoch"):
        assert t[f].tolist() == v[f], f
    assert h["lane_bytes"][: v["n_lanes"]].tolist() == v["lane_bytes"]
    assert h["total_tiles"] == v["total_tiles"] and h["flags"] == v["flags"]
    if len(v["credits"]) == 1:  # the same row passed by value instead of through device memory
        kw["credits"] = v["credits"][0]
        sched2 = core.schedule(**kw)
        torch.cuda.synchronize()
        assert sched2.table_numpy().tobytes() == t.tobytes()


# ---- staging windows on HIP VMM ------------------------------------------------------------------------------
def test_pool_windows_first_fit_and_exhaustion(fl):
    core, torch = fl
    pool = core.Pool(0, 16)
    gran = pool.granularity()
    assert gran > 0 and (2 * MB) % gran == 0 or gran % (2 * MB) == 0
    assert pool.free_units() == 16
    a = core.Window(pool, 10 * MB)
    b = core.Window(pool, 64 * MB)
    a.bind(5 * MB)                        # ceil(5 MiB / 2 MiB) = 3 units, first free slots first (cumem.cu:157-175)
    assert a.slots() == [0, 1, 2] and a.bound_bytes == 6 * MB and pool.free_units() == 13
    b.bind(2 * MB)
    assert b.slots() == [3]
    a.trim(2 * MB)                        # gives slots 1 and 2 back
    assert a.slots() == [0] and pool.free_units() == 14
    b.bind(6 * MB)                        # takes the lowest free slots again
    assert b.slots() == [3, 1, 2]
    assert pool.slot_of(b.base + 2 * MB) == 1 and pool.slot_of(a.base) == 0
    # data written through the window lands and survives
    n = 6 * MB
    src = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda")
    core.check(core._lib.load().flh_copy(C.c_void_p(b.base), C.c_void_p(src.data_ptr()), n, None))
    torch.cuda.synchronize()
    assert torch.equal(core.read_window(b.base, n), src)
    # exhaustion: 16 units in the pool, 4 in use
    with pytest.raises(core._lib.FuseLinkError) as e:
        b.bind(64 * MB)
    assert e.value.code == -4             # FLH_E_NOMEM; what was bound before the failure stays bound (cumem.cu:176-179)
    assert pool.free_units() == 0 and len(b.slots()) == 15
    with pytest.raises(core._lib.FuseLinkError):
        a.bind(11 * MB)                   # beyond the reserved range
    with pytest.raises(core._lib.FuseLinkError):
        pool.destroy()                    # windows still alive
    a.destroy(), b.destroy()
    assert pool.free_units() == 16
    pool.destroy()


def test_window_units_export_as_dmabuf(fl):
    """What a NIC driver needs to read a lane's staged bytes (ibv_reg_dmabuf_mr in src/plugin.cc:1278-1280):
    a DMA-BUF descriptor for bound units of a staging window."""
    import os
    import stat
    core, torch = fl
    pool = core.Pool(0, 8)
    w = core.Window(pool, 8 * MB)
    w.bind(4 * MB)
    fds = []
    try:
        fds.append(w.export_dmabuf(0, 2 * MB))            # one unit
        fds.append(w.export_dmabuf(2 * MB, 2 * MB))       # the next one
        for fd in fds:
            assert fd > 2
            st = os.fstat(fd)
            assert not stat.S_ISREG(st.st_mode) and not stat.S_ISDIR(st.st_mode)   # an anonymous dma-buf inode
        with pytest.raises(core._lib.FuseLinkError) as e:
            w.export_dmabuf(4 * MB, 2 * MB)                 # not bound
        assert e.value.code == -5
        with pytest.raises(core._lib.FuseLinkError):
            w.export_dmabuf(4096, 2 * MB)                   # not on a unit boundary
        with pytest.raises(core._lib.FuseLinkError):
            w.export_dmabuf(0, 4 * MB)                      # a descriptor covers one unit
        for fd in fds:
            assert os.fstat(fd).st_size == 2 * MB
        # the window still works after the export
        src = torch.randint(0, 255, (4 * MB,), dtype=torch.uint8, device="cuda")
        core.check(core._lib.load().flh_copy(C.c_void_p(w.base), C.c_void_p(src.data_ptr()), 4 * MB, None))
        torch.cuda.synchronize()
        assert torch.equal(core.read_window(w.base, 4 * MB), src)
    finally:
        for fd in fds:
            os.close(fd)
    w.destroy()
    pool.destroy()


def test_region_refcount_translate_and_mirror_mode(fl):
    core, torch = fl
    pool = core.Pool(0, 64)
    buf = torch.randint(0, 255, (8 * MB + 4096,), dtype=torch.uint8, device="cuda")
    base, nbytes = buf.data_ptr(), buf.numel()
    r1 = core.Region(pool, base, nbytes, 4, nbytes)
    r2 = core.Region(pool, base, nbytes, 4, nbytes)       # same base: shared, counted (plugin.cc:1214-1226)
    assert r1.handle_value == r2.handle_value and r1.refs() == 2
    w = r1.windows()
    assert w.n_lanes == 4 and all(w.cap[l] >= nbytes for l in range(4))
    units = (nbytes + 2 * MB - 1) // (2 * MB)
    assert pool.free_units() == 64 - 4 * units
    # pointer translation: window + (data - start_addr) (plugin.cc:1582, 1626)
    for lane in range(4):
        for off in (0, 1, 4096, nbytes - 1):
            assert r1.translate(lane, base + off) == w.base[lane] + off
    assert r1.translate(0, base + nbytes) == 0 and r1.translate(9, base) == 0
    # mirror mode: every chunk sits in its lane's window at the offset it has in the user buffer
    chunk = 256 << 10
    sched = core.schedule(n_lanes=4, credits=[1, 2, 3, 4], quantum=chunk, total_bytes=nbytes, chunk_bytes=chunk,
                          mode=core.SCHED_MIRROR)
    status = core.new_status()
    core.stripe(buf, w, sched, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    t = sched.table_numpy()
    host = buf.cpu().numpy()
    for i in (0, 1, 7, len(t) - 1):
        staged = core.read_window(r1.translate(int(t["lane"][i]), base + int(t["src_off"][i])), int(t["len"][i])).cpu().numpy()
        np.testing.assert_array_equal(staged, host[int(t["src_off"][i]): int(t["src_off"][i]) + int(t["len"][i])])
    dst = torch.zeros_like(buf)
    core.reassemble(dst, w, sched, status)
    torch.cuda.synchronize()
    assert torch.equal(dst, buf)
    assert r2.release() == 1 and pool.free_units() == 64 - 4 * units
    assert r1.release() == 0 and pool.free_units() == 64   # destroyed with the last reference (plugin.cc:1382-1403)
    pool.destroy()


# ---- expert-parallel send set: 256 variable blocks of 7168-wide bf16 rows --------------------------------
def _zipf_rows(rng, n, s=1.1, cap=4096):
    ranks = np.arange(1, cap + 1, dtype=np.float64)
    p = ranks ** (-s)
    p /= p.sum()
    return rng.choice(np.arange(1, cap + 1), size=n, p=p)


def test_cfg3_expert_parallel_send_set(fl):
    core, torch = fl
    rng = np.random.default_rng(3)
    rows = _zipf_rows(rng, 256)
    row_bytes = 7168 * 2
    sizes = (rows * row_bytes).astype(np.uint32)
    total = int(sizes.sum())
    credits = np.array([4, 4, 4, 4, 4, 4, 4, 1], dtype=np.uint32)      # one lane at 25 % idleness
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    src = torch.randint(-32768, 32767, (total // 2,), dtype=torch.int16, device="cuda", generator=gen).view(torch.uint8)
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=8, credits=credits, quantum=256 << 10, sizes=sizes)
    sched = core.schedule(n_lanes=8, credits=_dev(torch, credits.view(np.int32)), quantum=256 << 10,
                          sizes=_dev(torch, sizes.view(np.int32)))
    torch.cuda.synchronize()
    got_t, got_h = sched.table_numpy(), sched.hdr_numpy()
    assert got_t.tobytes() == exp_t.tobytes()
    np.testing.assert_array_equal(got_h["lane_bytes"], exp_h["lane_bytes"])
    caps = [int(b) for b in exp_h["lane_bytes"][:8]]
    wins = [torch.zeros(max(c, 1), dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    dst = torch.zeros_like(src)
    core.stripe(src, w, sched, status)
    core.reassemble(dst, w, sched, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and torch.equal(src, dst)
    # windows against the host-memcpy windows for the three largest and three smallest blocks' lanes
    src_np = src.cpu().numpy()
    exp_w = ob.cpu_stripe(src_np, exp_t, caps)
    for l in range(8):
        np.testing.assert_array_equal(wins[l].cpu().numpy()[: caps[l]], exp_w[l][: caps[l]])


# ---- paged KV-cache gather --------------------------------------------------------------------------------------
@pytest.mark.parametrize("by_lane", [False, True])
@pytest.mark.parametrize("use_lds", [False, True])
def test_cfg4_paged_kv_gather(fl, use_lds, by_lane):
    core, torch = fl
    rng = np.random.default_rng(4)
    n_pages, page = 4096, 16 * 8 * 128 * 2            # 32 KiB pages: 16 tokens x 8 KV heads x 128 dim bf16
    ppc, chunk = 4, 4 * page                          # 128 KiB chunks
    gen = torch.Generator(device="cuda")
    for name, seed in (("K", 41), ("V", 42)):
        gen.manual_seed(seed)
        pool = torch.randint(-32768, 32767, (n_pages * page // 2,), dtype=torch.int16, device="cuda", generator=gen).view(torch.uint8)
        table_np = rng.permutation(n_pages).astype(np.uint32)
        table = _dev(torch, table_np.view(np.int32))
        credits = rng.integers(1, 9, size=8).astype(np.uint32)
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=8, credits=credits, quantum=chunk, total_bytes=n_pages * page, chunk_bytes=chunk)
        sched = core.schedule(n_lanes=8, credits=_dev(torch, credits.view(np.int32)), quantum=chunk,
                              total_bytes=n_pages * page, chunk_bytes=chunk, by_lane=by_lane)
        torch.cuda.synchronize()
        assert sched.table_numpy().tobytes() == exp_t.tobytes()
        caps = [int(b) for b in exp_h["lane_bytes"][:8]]
        wins = [torch.zeros(max(c, 1), dtype=torch.uint8, device="cuda") for c in caps]
        w = core.make_windows([t.data_ptr() for t in wins], caps)
        status = core.new_status()
        core.gather_pages(pool, table, page, ppc, w, sched, status, use_lds=use_lds, by_lane=by_lane)
        out = torch.zeros_like(pool)
        core.scatter_pages(out, table, page, ppc, w, sched, status, use_lds=use_lds)
        torch.cuda.synchronize()
        assert int(status.item()) == 0
        assert torch.equal(out, pool), name
        # the staged windows hold the pages in table order, as an index-by-index CPU gather puts them
        pool_np = pool.cpu().numpy()
        exp_w = ob.cpu_gather_pages(pool_np, table_np, page, ppc, exp_t, caps)
        for l in range(8):
            np.testing.assert_array_equal(wins[l].cpu().numpy()[: caps[l]], exp_w[l][: caps[l]])


@pytest.mark.parametrize("seed", range(16))
def test_fused_paged_gather_equals_oracle(fl, seed):
    """flh_gather_pages_uniform / flh_scatter_pages_uniform: the table the gather writes, the staged windows and
    the scattered pool against the oracle; page sizes that are and are not powers of two, a ragged last chunk,
    a pool larger than the message, carried epoch bytes, destination order."""
    core, torch = fl
    rng = np.random.default_rng(7000 + seed)
    lanes = int(rng.integers(1, 17))
    page = int(rng.choice([256, 4096, 4096 + 512, 32768]))
    tile = page if page <= 32768 else 32768
    ppc = int(rng.integers(1, 6))
    n_pages = int(rng.integers(1, 300))
    pool_pages = n_pages + int(rng.integers(0, 20))
    total, chunk = n_pages * page, ppc * page
    credits = rng.integers(0, 9, size=lanes).astype(np.uint32)
    if seed == 1:
        credits[:] = 0
    epoch_bytes = int(rng.integers(0, 30)) * chunk
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["epoch_bytes"] = epoch_bytes
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                         mode=1, state=st, tile_bytes=tile)
    caps = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    pool_np = rng.integers(0, 256, size=pool_pages * page, dtype=np.uint8)
    table_np = rng.permutation(pool_pages).astype(np.uint32)[:n_pages]
    padded = np.concatenate([table_np, np.zeros((-n_pages) % ppc, dtype=np.uint32)])
    exp_w = ob.cpu_gather_pages(pool_np, padded, page, ppc, exp_t, caps)
    pool = _dev(torch, pool_np)
    table = _dev(torch, table_np.view(np.int32))
    u = core.uniform_params(total, chunk, credits.tolist(), epoch_bytes=epoch_bytes, tile_bytes=tile)
    for dest_order in (0, 1):
        wins = [torch.zeros(max(c, 1), dtype=torch.uint8, device="cuda") for c in caps]
        w = core.make_windows([t.data_ptr() for t in wins], caps)
        out = core.new_schedule_buffers(len(exp_t), tile_bytes=tile)
        status = core.new_status()
        core.tune("stripe_dest_order", dest_order)
        try:
            core.gather_pages_uniform(pool, table, page, w, u, status, out=out)
        finally:
            core.tune("stripe_dest_order", -1)
        back = torch.zeros_like(pool)
        core.scatter_pages_uniform(back, table, page, w, u, status)
        torch.cuda.synchronize()
        assert int(status.item()) == 0
        got_t = out.table_numpy()
        for f in ob.DESC_DTYPE.names:
            np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f"table field {f}")
        for l in range(lanes):
            np.testing.assert_array_equal(wins[l].cpu().numpy()[: caps[l]], exp_w[l][: caps[l]], err_msg=f"lane {l}")
        # the pages the table names came back; every other page of the pool stayed untouched (zero)
        back_np = back.cpu().numpy().reshape(pool_pages, page)
        named = np.zeros(pool_pages, dtype=bool)
        named[table_np] = True
        np.testing.assert_array_equal(back_np[named], pool_np.reshape(pool_pages, page)[named])
        assert not back_np[~named].any()


def test_fused_paged_gather_refuses_what_it_cannot_name(fl):
    core, torch = fl
    page, lanes = 4096, 2
    pool = torch.zeros(8 * page, dtype=torch.uint8, device="cuda")
    wins = [torch.zeros(8 * page, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
    w = core.make_windows([t.data_ptr() for t in wins], [8 * page] * lanes)
    status = core.new_status()
    good = _dev(torch, np.arange(8, dtype=np.int32))
    with pytest.raises(Exception):   # a tile would straddle pages
        core.gather_pages_uniform(pool, good, page, w, core.uniform_params(8 * page, 2 * page, [1, 1], tile_bytes=8192), status)
    with pytest.raises(Exception):   # chunks that are not whole pages
        core.gather_pages_uniform(pool, good, page, w, core.uniform_params(8 * page, page + 128, [1, 1], tile_bytes=128), status)
    bad = _dev(torch, np.array([0, 1, 2, 3, 4, 5, 6, 99], dtype=np.int32))   # page 99 is not in the pool
    core.gather_pages_uniform(pool, bad, page, w, core.uniform_params(8 * page, 2 * page, [1, 1], tile_bytes=4096), status)
    torch.cuda.synchronize()
    assert int(status.item()) == -5   # FLH_E_RANGE


def test_paged_gather_with_more_chunks_than_the_grid_is_tall(fl):
    """70 000 one-page chunks: the page kernels' grid is at most 65 535 chunks tall and steps over the rest."""
    core, torch = fl
    rng = np.random.default_rng(15)
    n_pages, page, ppc = 70000, 256, 1
    total = n_pages * page
    pool = torch.randint(0, 255, (total,), dtype=torch.uint8, device="cuda")
    table_np = rng.permutation(n_pages).astype(np.uint32)
    credits = np.array([2, 1, 3, 1], dtype=np.uint32)
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=4, credits=credits, quantum=page, total_bytes=total, chunk_bytes=page)
    sched = core.schedule(n_lanes=4, credits=credits.tolist(), quantum=page, total_bytes=total, chunk_bytes=page)
    caps = [int(b) for b in exp_h["lane_bytes"][:4]]
    wins = [torch.zeros(c, dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    table = _dev(torch, table_np.view(np.int32))
    core.gather_pages(pool, table, page, ppc, w, sched, status)
    out = torch.zeros_like(pool)
    core.scatter_pages(out, table, page, ppc, w, sched, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and torch.equal(out, pool)
    exp_w = ob.cpu_gather_pages(pool.cpu().numpy(), table_np, page, ppc, exp_t, caps)
    for l in range(4):
        np.testing.assert_array_equal(wins[l].cpu().numpy()[: caps[l]], exp_w[l][: caps[l]])


def test_paged_gather_ragged_and_bad_page(fl):
    core, torch = fl
    rng = np.random.default_rng(14)
    n_pages, page, ppc = 37, 4096 + 512, 4            # odd page size, last chunk holds one page
    total = n_pages * page
    pool = torch.randint(0, 255, (n_pages * page,), dtype=torch.uint8, device="cuda")
    table_np = rng.permutation(n_pages).astype(np.uint32)
    table_np = np.concatenate([table_np, np.zeros(3, dtype=np.uint32)])   # padded to whole chunks
    credits = np.array([1, 3, 2], dtype=np.uint32)
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=3, credits=credits, quantum=page * ppc, total_bytes=total, chunk_bytes=page * ppc)
    sched = core.schedule(n_lanes=3, credits=[1, 3, 2], quantum=page * ppc, total_bytes=total, chunk_bytes=page * ppc, by_lane=True)
    caps = [int(b) for b in exp_h["lane_bytes"][:3]]
    wins = [torch.zeros(max(c, 1) + 32, dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    table = _dev(torch, table_np.view(np.int32))
    for lds, by_lane in ((False, False), (True, False), (False, True), (True, True)):
        for t in wins:
            t.zero_()
        core.gather_pages(pool, table, page, ppc, w, sched, status, use_lds=lds, by_lane=by_lane)
        out = torch.zeros_like(pool)
        core.scatter_pages(out, table, page, ppc, w, sched, status, use_lds=lds)
        torch.cuda.synchronize()
        assert int(status.item()) == 0 and torch.equal(out, pool)
        exp_w = ob.cpu_gather_pages(pool.cpu().numpy(), table_np, page, ppc, exp_t, caps)
        for l in range(3):
            got = wins[l].cpu().numpy()
            np.testing.assert_array_equal(got[: caps[l]], exp_w[l][: caps[l]])
            assert not got[caps[l]:].any()
    # a page number outside the pool is refused, not read
    bad = table_np.copy()
    bad[5] = 10_000
    core.gather_pages(pool, _dev(torch, bad.view(np.int32)), page, ppc, w, sched, status)
    torch.cuda.synchronize()
    assert int(status.item()) == -5


# ---- stress: 1 GiB, 64 KiB chunks, 16 lanes, credits redrawn every 1000 chunks -----------------------------------
def test_cfg2_fused_pair_stages_the_oracles_windows(fl):
    """The bench's default path at its full size: 64 MiB fp16 N(0,1), 256 KiB chunks, 8 lanes, credits seeded in [1,8],
    through flh_stripe_uniform / flh_reassemble_uniform.  All eight staging windows byte for byte against the oracle's
    host-memcpy windows, the table and header the striping launch writes against the oracle's, the reassembled buffer
    against the source."""
    core, torch = fl
    rng = np.random.default_rng(2)
    total, chunk, lanes = 64 << 20, 256 << 10, 8
    credits = rng.integers(1, 9, size=lanes).astype(np.uint32)
    src_np = rng.standard_normal(total // 2, dtype=np.float32).astype(np.float16).view(np.uint8)
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                         mode=ob.SCHED_RESET_OFFSETS)
    lane_bytes = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    exp_w = ob.cpu_stripe(src_np, exp_t, lane_bytes)
    pool = core.Pool(0, sum((b + 2 * MB - 1) // (2 * MB) for b in lane_bytes))
    wins = []
    for b in lane_bytes:
        w = core.Window(pool, b)
        w.bind(b)
        wins.append(w)
    win = core.make_windows([w.base for w in wins], [w.bound_bytes for w in wins])
    src = _dev(torch, src_np)
    dst = torch.zeros_like(src)
    u = core.uniform_params(total, chunk, credits.tolist())
    out = core.new_schedule_buffers(len(exp_t))
    status = core.new_status()
    core.stripe_uniform(src, win, u, status, out=out)
    core.reassemble_uniform(dst, win, u, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    assert out.table_numpy().tobytes() == exp_t.tobytes()
    got_h = out.hdr_numpy()
    for f in ("total_bytes", "total_tiles", "n_chunks", "flags", "uniform_tiles", "lane_bytes", "lane_chunks"):
        np.testing.assert_array_equal(got_h[f], exp_h[f], err_msg=f)
    for l in range(lanes):
        got = core.read_window(wins[l].base, lane_bytes[l]).cpu().numpy()
        assert got.tobytes() == exp_w[l][: lane_bytes[l]].tobytes(), f"staging window {l} differs from the host-memcpy window"
    assert torch.equal(src, dst)
    for w in wins:
        w.destroy()
    pool.destroy()


def test_cfg5_stress_full_size(fl):
    core, torch = fl
    rng = np.random.default_rng(5)
    total, chunk, lanes, E = 1 << 30, 64 << 10, 16, 1000
    n = total // chunk
    rows = (n + E - 1) // E
    credits = rng.integers(1, 9, size=(rows, lanes)).astype(np.uint32)
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk, epoch_len=E)
    sched = core.schedule(n_lanes=lanes, credits=_dev(torch, credits.view(np.int32)), quantum=chunk, total_bytes=total,
                          chunk_bytes=chunk, epoch_len=E)
    torch.cuda.synchronize()
    assert sched.table_numpy().tobytes() == exp_t.tobytes()           # 16384-row chunk -> lane table, bit-exact
    got_h = sched.hdr_numpy()
    np.testing.assert_array_equal(got_h["lane_bytes"], exp_h["lane_bytes"])
    assert got_h["lane_bytes"].sum() == total
    lane_bytes = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    units = sum((b + 2 * MB - 1) // (2 * MB) for b in lane_bytes)
    pool = core.Pool(0, units)
    wins = []
    for b in lane_bytes:
        w = core.Window(pool, b)
        w.bind(b)
        wins.append(w)
    assert pool.free_units() == 0
    win = core.make_windows([w.base for w in wins], [w.bound_bytes for w in wins])
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    src = torch.randint(0, 2**31 - 1, (total // 4,), dtype=torch.int32, device="cuda", generator=gen).view(torch.uint8)
    dst = torch.zeros_like(src)
    status = core.new_status()
    hint = core.uniform_hint(total, chunk)
    core.stripe(src, win, sched, status, hint=hint)
    core.reassemble(dst, win, sched, status, hint=hint)
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and torch.equal(src, dst)
    # spot-check staged chunks against the table: first, last, and a few in the middle
    src_np = src[: 4 * chunk].cpu().numpy()
    for i in (0, 1, 2, 3):
        got = core.read_window(wins[int(exp_t["lane"][i])].base + int(exp_t["win_off"][i]), chunk).cpu().numpy()
        np.testing.assert_array_equal(got, src_np[i * chunk: (i + 1) * chunk])
    for i in (999, 1000, 8191, n - 1):
        got = core.read_window(wins[int(exp_t["lane"][i])].base + int(exp_t["win_off"][i]), chunk)
        assert torch.equal(got, src[i * chunk: (i + 1) * chunk])
    for w in wins:
        w.destroy()
    pool.destroy()


def test_message_beyond_4_gib(fl):
    """Offsets past 2^32: a 4 GiB + 3 MiB + 5 B message over 8 lanes through the table-driven kernels (chunk order
    and destination order), the fused kernels (which pick destination order by themselves at this size) and the
    generic tile-search kernel; the table against the oracle, the round trip bit for bit."""
    core, torch = fl
    total, chunk, lanes = (4 << 30) + (3 << 20) + 5, 1 << 20, 8
    credits = [5, 1, 7, 2, 8, 3, 1, 6]
    free, _ = torch.cuda.mem_get_info()
    if free < 4 * total:
        pytest.skip("not enough device memory for three 4 GiB buffers")
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk)
    assert int(exp_t["src_off"][-1]) > 2**32 and int(exp_h["lane_bytes"].max()) < 2**32
    gen = torch.Generator(device="cuda")
    gen.manual_seed(44)
    src = torch.randint(0, 2**31 - 1, ((total + 3) // 4,), dtype=torch.int32, device="cuda", generator=gen).view(torch.uint8)[:total]
    dst = torch.empty_like(src)
    sched = core.schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk, by_lane=True)
    torch.cuda.synchronize()
    assert sched.table_numpy().tobytes() == exp_t.tobytes()
    caps = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    wins = [torch.empty(c, dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    hint = core.uniform_hint(total, chunk)
    u = core.uniform_params(total, chunk, credits)

    def check(tag):
        torch.cuda.synchronize()
        assert int(status.item()) == 0, tag
        assert torch.equal(src, dst), tag
        dst.zero_()
        for t in wins:
            t.zero_()

    dst.zero_()
    core.stripe(src, w, sched, status, hint=hint)
    core.reassemble(dst, w, sched, status, hint=hint)
    check("table-driven, chunk order")
    core.stripe(src, w, sched, status, hint=hint, by_lane=True)
    core.reassemble(dst, w, sched, status, hint=hint)
    check("table-driven, destination order")
    core.stripe(src, w, sched, status)          # no host hint: the tile-search kernel
    core.reassemble(dst, w, sched, status)
    check("generic kernel")
    out = core.new_schedule_buffers(len(exp_t))
    core.stripe_uniform(src, w, u, status, out=out)
    core.reassemble_uniform(dst, w, u, status)
    check("fused")
    assert out.table_numpy().tobytes() == exp_t.tobytes()
