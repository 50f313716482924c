"""Pins the CPU oracle: hand-worked vectors (tests/golden), the reference's own monitor client
compiled from src/monitor.h (oracle/_ref), invariants and brute force on tiny inputs.  A plausible
slip in the oracle (dropped term, wrong index, off-by-one at the timeout) fails one of these."""
import ctypes as C
import itertools
import json
import os

import numpy as np
import pytest

from tests import oracle_binding as ob

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat_vectors.json")))
L = ob.lib()


# ---- R1 / R2 / R3 / R4 ------------------------------------------------------------------------------
@pytest.mark.parametrize("v", KAT["split"])
def test_split_vectors(v):
    off, ln = ob.split(v["nbytes"], v["chunk"])
    assert off == v["off"] and ln == v["len"]


def test_split_invariants():
    rng = np.random.default_rng(0)
    for _ in range(300):
        n = int(rng.integers(0, 1 << 26))
        c = int(rng.integers(1, 1 << 20))
        off, ln = ob.split(n, c)
        assert sum(ln) == n
        assert all(off[i + 1] == off[i] + ln[i] for i in range(len(off) - 1))
        assert all(x == c for x in ln[:-1]) and (not ln or 0 < ln[-1] <= c)


@pytest.mark.parametrize("v", KAT["step_size"])
def test_step_size(v):
    assert L.fl_step_size(v["buffsize"], v["steps"], v["p2p_chunk"]) == v["expect"]


@pytest.mark.parametrize("v", KAT["qp_split"])
def test_qp_split_vectors(v):
    assert ob.qp_split(v["size"], v["nqps"]) == (v["stride"], v["off"], v["len"])


def test_qp_split_invariants():
    rng = np.random.default_rng(1)
    for _ in range(500):
        size = int(rng.integers(0, 1 << 22))
        nqps = int(rng.integers(1, 17))
        stride, off, ln = ob.qp_split(size, nqps)
        assert sum(ln) == size and all(o % 128 == 0 for o in off) and stride % 128 == 0
        assert all(l >= 0 for l in ln)
    assert ob.qp_split(12345, 1) == (12416, [0], [12345])  # one QP, the default (src/plugin.cc:584): identity


def test_lane_static_brute_force():
    for nics in range(1, 17):
        for cid in range(1024):
            assert L.fl_lane_static(cid, nics) == cid % nics


def test_refresh_cadence_sets():
    rx = [k for k in range(64) if L.fl_refresh_rx_due(k, 5, 5)]
    tx = [k for k in range(64) if L.fl_refresh_tx_due(k)]
    assert rx == [0, 8, 16, 24, 32, 40, 48, 56]      # n_finished % 8 == 0 (src/plugin.cc:1700)
    assert tx == [7, 15, 23, 31, 39, 47, 55, 63]     # (n_finished + 1) % 8 == 0 (src/plugin.cc:1443)
    assert not L.fl_refresh_rx_due(8, 6, 5)          # something received is not consumed yet (src/plugin.cc:1704-1709)


# ---- R5: monitor ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("v", KAT["monitor_timeout"])
def test_monitor_timeout_vectors(v):
    m = ob.Monitor()
    L.fl_mon_init(C.byref(m))
    L.fl_mon_mark_tx(C.byref(m), 3, 0, v["mark_at"])
    L.fl_mon_mark_rx(C.byref(m), 5, 0, v["mark_at"])
    assert m.tx_status[3] == 1 and m.tx_last_active[3] == v["mark_at"]
    L.fl_mon_tick(C.byref(m), v["tick_at"])
    assert m.tx_status[3] == v["status"] and m.rx_status[5] == v["status"]


@pytest.mark.parametrize("v", KAT["idle_pick"])
def test_idle_pick_vectors(v):
    m = ob.Monitor()
    L.fl_mon_init(C.byref(m))
    arr = m.tx_status if v["dir"] == "tx" else m.rx_status
    for i, s in enumerate(v["status"]):
        arr[i] = s
    ret = L.fl_mon_idle_pick_tx(C.byref(m), v["group"]) if v["dir"] == "tx" else L.fl_mon_idle_pick_rx(C.byref(m), v["group"], v["mask"])
    assert ret == v["ret"] and list(arr) == v["after"]


def _ref_monitor():
    path = os.path.join(ob.ORACLE_DIR, "_ref", "libref_monitor.so")
    if not os.path.exists(path):
        pytest.skip("oracle/_ref/libref_monitor.so not built (the reference tree is not present)")
    ref = C.CDLL(path)
    ref.ref_mon_set.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_longlong]
    ref.ref_mon_get_ts.restype = C.c_longlong
    ref.ref_mon_now.restype = C.c_longlong
    if ref.ref_mon_open() != 0:
        pytest.skip("POSIX shared memory or semaphores are not available here")
    return ref


def test_monitor_constants_and_layout_match_reference_header():
    ref = _ref_monitor()
    try:
        c = [ref.ref_mon_const(i) for i in range(14)]
        assert c[0:5] == [16, 1, 16, 2, 160]          # MAX_NIC_NUM, NNIC_PER_GROUP, NGROUP, NCHANNELS_PER_NIC, timeout
        assert c[5:8] == [0, 1, 2]                    # IDLE, BUSY, BORROWED
        assert c[9:13] == [0, 64, 128, 256]           # two int[16][1] status arrays, then two int64[16][1] timestamp arrays
        assert c[13] == 384 and c[8] >= 385
        assert C.sizeof(ob.Monitor) == 384
    finally:
        ref.ref_mon_close()


def test_idle_pick_and_mark_against_reference_client():
    """Every idle/busy/borrowed pattern over 6 groups, every own-group, a few masks: the restated
    getIdleNicTx/Rx must return the same NIC and leave the same statuses as the reference's class."""
    ref = _ref_monitor()
    try:
        rng = np.random.default_rng(3)
        patterns = list(itertools.product([0, 1, 2], repeat=5))
        for pat in patterns[::3]:
            status = list(pat) + [int(x) for x in rng.integers(0, 3, size=11)]
            for group in (0, 2, 15):
                for tx, mask in ((1, -1), (0, 0xFFFF), (0, int(rng.integers(0, 1 << 16))), (0, 0)):
                    m = ob.Monitor()
                    L.fl_mon_init(C.byref(m))
                    for i, s in enumerate(status):
                        ref.ref_mon_set(tx, i, 0, s, 0)
                        (m.tx_status if tx else m.rx_status)[i] = s
                    got = L.fl_mon_idle_pick_tx(C.byref(m), group) if tx else L.fl_mon_idle_pick_rx(C.byref(m), group, mask)
                    exp = ref.ref_mon_idle_pick_tx(group, 0) if tx else ref.ref_mon_idle_pick_rx(group, 0, mask)
                    assert got == exp, (status, group, tx, mask)
                    after = [ref.ref_mon_get_status(tx, i, 0) for i in range(16)]
                    assert list(m.tx_status if tx else m.rx_status) == after
        # mark: timestamp from the steady clock, status BUSY (src/monitor.h:236-250)
        for tx in (0, 1):
            ref.ref_mon_set(tx, 4, 0, 2, 0)
            t0 = ref.ref_mon_now()
            (ref.ref_mon_mark_tx if tx else ref.ref_mon_mark_rx)(4, 0)
            t1 = ref.ref_mon_now()
            assert ref.ref_mon_get_status(tx, 4, 0) == 1 and t0 <= ref.ref_mon_get_ts(tx, 4, 0) <= t1
        out = (C.c_int * 16)()
        for i in range(16):
            ref.ref_mon_set(1, i, 0, i % 3, 0)
        ref.ref_mon_status(16, out)
        m = ob.Monitor()
        for i in range(16):
            m.tx_status[i] = i % 3
        mine = (C.c_int32 * 16)()
        L.fl_mon_status(C.byref(m), 16, mine)
        assert list(out) == list(mine)
    finally:
        ref.ref_mon_close()


def test_credits_from_status():
    st = (C.c_int32 * 4)(0, 1, 2, 0)
    out = (C.c_uint32 * 4)()
    L.fl_credits_from_status(st, 4, 1, 4, out)
    assert list(out) == [4, 1, 0, 4]   # idle -> 4, busy own lane -> 1, borrowed -> 0
    L.fl_credits_from_status(st, 4, 3, 2, out)
    assert list(out) == [2, 0, 0, 2]


def test_tx_usage_mask_and_rx_credits():
    """The content of the reference's placeholder mask (refreshTxUsage, fuselink.h:261-267) and what the receiver makes of
    it (getIdleNicRx's mask, monitor.h:208-224).  Hand vectors; the all-idle table gives the placeholder's own value; an
    all-ones mask reduces the receiver's half to fl_credits_from_status; and every status pattern of four lanes against
    the definition evaluated in Python."""
    IDLE, BUSY, BORROWED = 0, 1, 2
    st = (C.c_int32 * 4)(IDLE, BUSY, BORROWED, IDLE)
    assert L.fl_tx_usage_mask(st, 4, 1) == 0xfffffffb          # lane 2 borrowed: out; lane 1 busy but the comm's own: in
    assert L.fl_tx_usage_mask(st, 4, 0) == 0xfffffff9
    assert L.fl_tx_usage_mask((C.c_int32 * 8)(), 8, 5) == 0xffffffff   # nothing busy: the placeholder's value (fuselink.h:262)
    out = (C.c_uint32 * 4)()
    L.fl_rx_credits_from_status(st, 4, 1, 4, 0xffffffff, out)
    assert list(out) == [4, 1, 0, 4]
    L.fl_rx_credits_from_status(st, 4, 1, 4, 0xfffffff6, out)   # the sender's lanes 0 and 3 are busy
    assert list(out) == [0, 1, 0, 0]
    L.fl_rx_credits_from_status(st, 4, 3, 2, 0xfffffff7, out)   # a masked own lane still keeps one credit
    assert list(out) == [2, 0, 0, 1]
    import itertools
    ref = (C.c_uint32 * 4)()
    for pattern in itertools.product((IDLE, BUSY, BORROWED), repeat=4):
        st = (C.c_int32 * 4)(*pattern)
        for own in (-1, 0, 2):
            exp_mask = 0xfffffff0
            for l, v in enumerate(pattern):
                if v == IDLE or l == own:
                    exp_mask |= 1 << l
            assert L.fl_tx_usage_mask(st, 4, own) == exp_mask
            L.fl_credits_from_status(st, 4, own, 3, ref)
            L.fl_rx_credits_from_status(st, 4, own, 3, 0xffffffff, out)
            assert list(out) == list(ref)
            for mask in (0x0, 0x5, 0xa, 0xf):
                L.fl_rx_credits_from_status(st, 4, own, 3, mask, out)
                exp = [3 if v == IDLE and (mask >> l) & 1 else 0 for l, v in enumerate(pattern)]
                if 0 <= own < 4 and exp[own] == 0:
                    exp[own] = 1
                assert list(out) == exp


# ---- R5: credit schedule ---------------------------------------------------------------------------------
def _run_sched_vector(v, fn):
    kw = dict(n_lanes=v["n_lanes"], credits=v["credits"], quantum=v["quantum"], epoch_len=v["epoch_len"], tile_bytes=v["tile_bytes"])
    if "sizes" in v:
        kw["sizes"] = v["sizes"]
    else:
        kw["total_bytes"], kw["chunk_bytes"] = v["total_bytes"], v["chunk_bytes"]
    return fn(**kw)


@pytest.mark.parametrize("v", KAT["schedule"], ids=[v["name"][:40] for v in KAT["schedule"]])
def test_schedule_vectors(v):
    t, h, _ = _run_sched_vector(v, ob.credit_schedule)
    for f in ("lane", "win_off", "src_off", "tile_base", "epoch"):
        assert t[f].tolist() == v[f], f
    assert h["lane_bytes"][: v["n_lanes"]].tolist() == v["lane_bytes"]
    assert h["total_tiles"] == v["total_tiles"] and h["flags"] == v["flags"]
    assert h["total_bytes"] == sum(t["len"].tolist())


def _naive_schedule(sizes, L_, credits, E, q):
    """The written definition, evaluated the slow way (independent of the C code)."""
    lanes, offs = [], []
    for i in range(len(sizes)):
        e = i // E if E else 0
        row = list(credits[e % len(credits)])
        if sum(row) == 0:
            row = [1] * L_
        P = sum(sizes[j] for j in range(i) if (j // E if E else 0) == e)
        slot = (P // q) % sum(row)
        lane = next(l for l in range(L_) if sum(row[:l]) <= slot < sum(row[: l + 1]))
        lanes.append(lane)
    for i in range(len(sizes)):
        offs.append(sum(sizes[j] for j in range(i) if lanes[j] == lanes[i]))
    return lanes, offs


def test_schedule_brute_force_tiny():
    rng = np.random.default_rng(4)
    for _ in range(400):
        n = int(rng.integers(1, 13))
        L_ = int(rng.integers(1, 5))
        rows = int(rng.integers(1, 4))
        credits = rng.integers(0, 4, size=(rows, L_))
        E = int(rng.choice([0, 1, 2, 3, 5]))
        q = int(rng.choice([1, 7, 16, 100]))
        sizes = rng.integers(0, 40, size=n) if rng.random() < 0.7 else np.full(n, q)
        t, h, _ = ob.credit_schedule(n_lanes=L_, credits=credits, quantum=q, sizes=sizes, epoch_len=E, tile_bytes=128)
        lanes, offs = _naive_schedule([int(s) for s in sizes], L_, credits.tolist(), E, q)
        assert t["lane"].tolist() == lanes and t["win_off"].tolist() == offs


def test_schedule_properties():
    rng = np.random.default_rng(5)
    for _ in range(100):
        L_ = int(rng.integers(1, 17))
        q = int(rng.choice([4096, 65536, 262144]))
        # (1) equal credits, quantum-sized chunks: the static policy lane = i mod L (src/fuselink.h:235)
        n = int(rng.integers(1, 300))
        t, h, _ = ob.credit_schedule(n_lanes=L_, credits=np.ones(L_), quantum=q, total_bytes=n * q, chunk_bytes=q)
        assert t["lane"].tolist() == [i % L_ for i in range(n)]
        # (2), (3), (4) on random credits
        credits = rng.integers(0, 9, size=L_)
        if credits.sum() == 0:
            credits[0] = 1
        W = int(credits.sum())
        rounds = int(rng.integers(1, 5))
        t, h, _ = ob.credit_schedule(n_lanes=L_, credits=credits, quantum=q, total_bytes=rounds * W * q, chunk_bytes=q)
        counts = np.bincount(t["lane"], minlength=L_)
        assert (counts == rounds * credits).all()                 # exactly c_l quanta per round of W
        assert (h["lane_bytes"][:L_] == counts * q).all() and h["lane_bytes"][:L_].sum() == rounds * W * q
        assert (counts[credits == 0] == 0).all()


def test_table_by_lane_is_a_stable_sort_with_the_last_lane_last():
    rng = np.random.default_rng(11)
    for _ in range(40):
        L_ = int(rng.integers(1, 17))
        chunk = int(rng.choice([4096, 65536, 100000]))
        n = int(rng.integers(1, 400))
        total = n * chunk - int(rng.integers(0, chunk))
        credits = rng.integers(0, 6, size=(int(rng.integers(1, 4)), L_))
        t, h, _ = ob.credit_schedule(n_lanes=L_, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                     epoch_len=int(rng.choice([0, 5, 64])))
        tpc = (chunk + 32767) // 32768
        got = ob.table_by_lane(t, L_, tpc)
        # independent statement: stable sort by the lane's distance behind the last chunk's lane
        key = (t["lane"].astype(np.int64) - int(t["lane"][-1]) - 1) % L_
        order = np.argsort(key, kind="stable")
        for f in ("src_off", "win_off", "len", "lane", "epoch"):
            np.testing.assert_array_equal(got[f], t[f][order])
        np.testing.assert_array_equal(got["tile_base"], np.arange(n, dtype=np.uint32) * tpc)
        # what the striping kernel relies on: the short chunk is the final row, windows are walked front to back
        assert got["len"][-1] == t["len"][-1] and (got["len"][:-1] == chunk).all()
        for l in range(L_):
            w = got["win_off"][got["lane"] == l]
            assert (np.diff(w.astype(np.int64)) == chunk).all()


def test_schedule_state_carry_equals_one_shot():
    rng = np.random.default_rng(6)
    sizes = rng.integers(0, 5000, size=500)
    credits = rng.integers(0, 5, size=(4, 6))
    for E in (0, 7, 64):
        whole, hw, sw = ob.credit_schedule(n_lanes=6, credits=credits, quantum=1024, sizes=sizes, epoch_len=E, tile_bytes=256)
        st = None
        parts, base = [], 0
        for lo, hi in ((0, 13), (13, 14), (14, 300), (300, 500)):
            t, h, st = ob.credit_schedule(n_lanes=6, credits=credits, quantum=1024, sizes=sizes[lo:hi], epoch_len=E,
                                          tile_bytes=256, state=st, src_base=base)
            base += int(sizes[lo:hi].sum())
            parts.append(t)
        cat = np.concatenate(parts)
        for f in ("src_off", "win_off", "len", "lane", "epoch"):
            assert (cat[f] == whole[f]).all(), f
        assert st["chunk_index"] == 500 and (st["lane_off"] == sw["lane_off"]).all()
    # mirror mode: the window offset is the buffer offset (src/plugin.cc:1582)
    t, _, _ = ob.credit_schedule(n_lanes=6, credits=credits, quantum=1024, sizes=sizes, mode=ob.SCHED_MIRROR, src_base=4096)
    assert (t["win_off"] == t["src_off"]).all() and t["src_off"][0] == 4096


# ---- R6 / R7 / R8 ----------------------------------------------------------------------------------------------
def test_geometry_vectors():
    g = KAT["geometry"]
    for size, gran, exp in g["align_up"]:
        assert L.fl_align_up(size, gran) == exp
    for size, unit, exp in g["window_units"]:
        assert L.fl_window_units(size, unit) == exp
    for base, data, start, exp in g["translate"]:
        assert L.fl_translate(base, data, start) == exp
    for gpu, ch, n, exp in g["relay_gpu"]:
        assert L.fl_relay_gpu(gpu, ch, n) == exp
    for data, size, page, addr, pages in g["page_span"]:
        a, p = C.c_uint64(), C.c_uint64()
        L.fl_page_span(data, size, page, C.byref(a), C.byref(p))
        assert (a.value, p.value) == (addr, pages)


def test_region_cache_refcount():
    c = ob.RegCache()
    L.fl_regcache_init(C.byref(c))
    assert [L.fl_regcache_reg(C.byref(c), 0x1000) for _ in range(3)] == [1, 2, 3]
    assert L.fl_regcache_reg(C.byref(c), 0x2000) == 1 and c.created == 2
    assert [L.fl_regcache_dereg(C.byref(c), 0x1000) for _ in range(3)] == [2, 1, 0]
    assert c.destroyed == 1 and L.fl_regcache_dereg(C.byref(c), 0x1000) == -1
    assert L.fl_regcache_reg(C.byref(c), 0x1000) == 1 and c.created == 3


def test_pool_first_fit_and_exhaustion():
    p = ob.Pool()
    L.fl_pool_init(C.byref(p))
    MB = 1 << 20
    slots = (C.c_int * 600)()
    assert L.fl_pool_register(C.byref(p), 0x10000000, 5 * MB, slots, 600) == 3 and list(slots[:3]) == [0, 1, 2]
    assert L.fl_pool_register(C.byref(p), 0x20000000, 2 * MB, slots, 600) == 1 and slots[0] == 3
    assert L.fl_pool_lookup(C.byref(p), 0x10000000 + 2 * MB) == 1
    assert L.fl_pool_release(C.byref(p), 0x10000000 + 2 * MB) == 1
    assert L.fl_pool_register(C.byref(p), 0x30000000, 4 * MB, slots, 600) == 2 and list(slots[:2]) == [1, 4]  # first fit
    assert L.fl_pool_lookup(C.byref(p), 0x12345) == -1
    q = ob.Pool()
    L.fl_pool_init(C.byref(q))
    assert L.fl_pool_register(C.byref(q), 0x40000000, 512 * MB, slots, 600) == 256 and list(slots[:256]) == list(range(256))
    assert L.fl_pool_register(C.byref(q), 0x80000000, 1, slots, 600) == -1      # the 257th unit (src/cumem.cu:176-179)
    r = ob.Pool()
    L.fl_pool_init(C.byref(r))
    assert L.fl_pool_register(C.byref(r), 0x40000000, 514 * MB, slots, 600) == -1 and sum(r.mapped) == 256


def test_request_table_and_fifo():
    t = ob.ReqTab()
    L.fl_reqtab_init(C.byref(t))
    assert [L.fl_reqtab_get(C.byref(t)) for _ in range(3)] == [0, 1, 2]
    L.fl_reqtab_free(C.byref(t), 1)
    assert L.fl_reqtab_get(C.byref(t)) == 1                                      # first free (src/plugin.cc:1070-1085)
    for _ in range(253):
        assert L.fl_reqtab_get(C.byref(t)) >= 0
    assert L.fl_reqtab_get(C.byref(t)) == -1                                     # 257th (src/plugin.cc:1082-1084)
    f = ob.Fifo()
    L.fl_fifo_init(C.byref(f))
    assert L.fl_fifo_match(C.byref(f)) == -1                                     # nothing posted: would block
    assert L.fl_fifo_post(C.byref(f)) == 0 and f.idx[0] == 1                     # idx = tail + 1 (src/plugin.cc:1632)
    assert L.fl_fifo_match(C.byref(f)) == 0 and L.fl_fifo_match(C.byref(f)) == -1
    for k in range(1, 600):
        assert L.fl_fifo_post(C.byref(f)) == k % 256
        assert L.fl_fifo_match(C.byref(f)) == k % 256


# ---- host striping baseline --------------------------------------------------------------------------------
def test_cpu_stripe_roundtrip_and_threads():
    rng = np.random.default_rng(8)
    src = rng.integers(0, 256, size=(4 << 20) + 17, dtype=np.uint8)
    t, h, _ = ob.credit_schedule(n_lanes=2, credits=[1, 1], quantum=512 << 10, total_bytes=src.size, chunk_bytes=512 << 10)
    caps = h["lane_bytes"][:2]
    w = ob.cpu_stripe(src, t, caps)
    # lane 0 holds chunks 0,2,4,6,8 back to back
    assert (w[0][: 512 << 10] == src[: 512 << 10]).all() and (w[0][512 << 10: 1 << 20] == src[1 << 20: 3 << 19]).all()
    assert (ob.cpu_reassemble(src.size, w, t) == src).all()
    med, best = ob.cpu_baseline(src, t, h, 2, threads=1, warm=1, iters=3)
    medm, _ = ob.cpu_baseline(src, t, h, 2, threads=2, warm=1, iters=3)
    assert 0 < best <= med and medm > 0


def test_cpu_paged_gather_scatter():
    rng = np.random.default_rng(9)
    page, ppc, n_pages = 256, 4, 64
    pool = rng.integers(0, 256, size=n_pages * page, dtype=np.uint8)
    table = rng.permutation(n_pages).astype(np.uint32)
    t, h, _ = ob.credit_schedule(n_lanes=3, credits=[1, 2, 1], quantum=page * ppc, total_bytes=n_pages * page, chunk_bytes=page * ppc)
    w = ob.cpu_gather_pages(pool, table, page, ppc, t, h["lane_bytes"][:3])
    c = 5
    k = 2
    got = w[t["lane"][c]][t["win_off"][c] + k * page: t["win_off"][c] + (k + 1) * page]
    assert (got == pool[table[c * ppc + k] * page: (table[c * ppc + k] + 1) * page]).all()
    back = ob.cpu_scatter_pages(pool.size, table, page, ppc, w, t)
    assert (back == pool).all()
