"""GPU parity of the scheduler and the striping / reassembly kernels against the CPU oracle.
All calls go through the C ABI of libnccl-net-fuselink.so (fuselink_amd.core is a ctypes shim)."""
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


def _check_schedule(fl, *, n_lanes, credits, quantum, sizes=None, total_bytes=0, chunk_bytes=0, epoch_len=0,
                    tile_bytes=32768, mode=0, state=None, src_off=None, src_base=0, workspace=False):
    core, torch = fl
    credits = np.asarray(credits, dtype=np.uint32).reshape(-1, n_lanes)
    exp_t, exp_h, exp_s = ob.credit_schedule(n_lanes=n_lanes, credits=credits, quantum=quantum, sizes=sizes,
                                             total_bytes=total_bytes, chunk_bytes=chunk_bytes, epoch_len=epoch_len,
                                             tile_bytes=tile_bytes, mode=mode, state=state, src_off=src_off,
                                             src_base=src_base)
    d_state = None
    if state is not None:
        d_state = _dev(torch, np.array([state], dtype=ob.STATE_DTYPE).view(np.uint8))
    sched = core.schedule(n_lanes=n_lanes, credits=_dev(torch, credits.view(np.int32)), quantum=quantum,
                          sizes=None if sizes is None else _dev(torch, np.asarray(sizes, dtype=np.uint32).view(np.int32)),
                          total_bytes=total_bytes, chunk_bytes=chunk_bytes, epoch_len=epoch_len, tile_bytes=tile_bytes,
                          mode=mode, state=d_state, src_base=src_base, workspace=workspace,
                          src_off=None if src_off is None else _dev(torch, np.asarray(src_off, dtype=np.uint64).view(np.int64)))
    torch.cuda.synchronize()
    got_t, got_h = sched.table_numpy(), sched.hdr_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f"table field {f}")
    for f in ("total_bytes", "total_tiles", "n_chunks", "flags", "uniform_tiles", "lane_bytes", "lane_chunks"):
        np.testing.assert_array_equal(got_h[f], exp_h[f], err_msg=f"hdr field {f}")
    if state is not None:
        got_s = core.state_numpy(d_state)
        for f in ob.STATE_DTYPE.names:
            np.testing.assert_array_equal(got_s[f], exp_s[f], err_msg=f"state field {f}")
    return sched, exp_t, exp_h


@pytest.mark.parametrize("n", [0, 1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 2049, 5000, 16384])
def test_schedule_uniform_sizes(fl, n):
    chunk = 65536
    total = n * chunk - (chunk // 3 if n else 0)
    rng = np.random.default_rng(n)
    _check_schedule(fl, n_lanes=8, credits=rng.integers(1, 9, size=8), quantum=chunk, total_bytes=total, chunk_bytes=chunk)


@pytest.mark.parametrize("seed", range(6))
def test_schedule_random_sizes_epochs(fl, seed):
    rng = np.random.default_rng(100 + seed)
    n = int(rng.integers(1, 6000))
    lanes = int(rng.integers(1, 17))
    rows = int(rng.integers(1, 40))
    sizes = rng.integers(0, 300000, size=n).astype(np.uint32)
    credits = rng.integers(0, 9, size=(rows, lanes)).astype(np.uint32)
    credits[rng.integers(0, rows)] = 0  # an all-busy epoch exercises the static fallback
    epoch_len = int(rng.choice([0, 1, 7, 8, 100, 1000]))
    quantum = int(rng.choice([4096, 65536, 100000, 262144]))
    _check_schedule(fl, n_lanes=lanes, credits=credits, quantum=quantum, sizes=sizes, epoch_len=epoch_len,
                    tile_bytes=int(rng.choice([4096, 32768])))


@pytest.mark.parametrize("lanes", [3, 16])
def test_schedule_credit_rows_summing_past_32_bits(fl, lanes):
    """Credits are u32 each, so a row may sum to 2^32 or more: the 64-bit prefixes must take over."""
    rng = np.random.default_rng(7 + lanes)
    credits = rng.integers(0, 9, size=(5, lanes)).astype(np.uint32)
    credits[1] = rng.integers(2**31, 2**32 - 1, size=lanes)  # W of this row needs more than 32 bits
    credits[3, 0] = 2**32 - 1
    sizes = rng.integers(1, 1 << 20, size=1500).astype(np.uint32)
    _check_schedule(fl, n_lanes=lanes, credits=credits, quantum=4096, sizes=sizes, epoch_len=100)
    _check_schedule(fl, n_lanes=lanes, credits=credits, quantum=65536, total_bytes=3000 * 65536 - 5, chunk_bytes=65536, epoch_len=100)


@pytest.mark.parametrize("seed", range(5))
def test_schedule_table_in_destination_order(fl, seed):
    core, torch = fl
    rng = np.random.default_rng(300 + seed)
    lanes = int(rng.integers(1, 17))
    rows = int(rng.integers(1, 20))
    chunk = int(rng.choice([4096, 65536, 98304]))
    n = int(rng.integers(1, 5000))
    total = n * chunk - int(rng.integers(0, chunk))
    epoch_len = int(rng.choice([0, 7, 1000]))
    credits = rng.integers(0, 9, size=(rows, lanes)).astype(np.uint32)
    exp_t, _, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                     epoch_len=epoch_len)
    exp = ob.table_by_lane(exp_t, lanes, (chunk + 32767) // 32768)
    sched = core.schedule(n_lanes=lanes, credits=_dev(torch, credits.view(np.int32)), quantum=chunk, total_bytes=total,
                          chunk_bytes=chunk, epoch_len=epoch_len, by_lane=True)
    torch.cuda.synchronize()
    got, got_t = sched.table_by_lane_numpy(), sched.table_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f"table field {f}")
        np.testing.assert_array_equal(got[f], exp[f], err_msg=f"by-lane field {f}")
    # both copies of the table move the same bytes
    lane_bytes = [int(b) for b in sched.hdr_numpy()["lane_bytes"][:lanes]]
    wins = [torch.zeros(max(b, 1), dtype=torch.uint8, device="cuda") for b in lane_bytes]
    w = core.make_windows([t.data_ptr() for t in wins], lane_bytes)
    src = torch.randint(0, 256, (total,), dtype=torch.uint8, device="cuda")
    status = core.new_status()
    for hint in (None, core.uniform_hint(total, chunk)):
        for t in wins:
            t.zero_()
        core.stripe(src, w, sched, status, hint=hint, by_lane=True)
        dst = torch.zeros_like(src)
        core.reassemble(dst, w, sched, status, hint=hint)
        torch.cuda.synchronize()
        assert int(status.item()) == 0 and torch.equal(src, dst)


def test_schedule_by_lane_needs_the_uniform_split(fl):
    core, torch = fl
    sizes = _dev(torch, np.full(10, 4096, dtype=np.int32))
    with pytest.raises(Exception):
        core.schedule(n_lanes=4, credits=[1, 1, 1, 1], quantum=4096, sizes=sizes, by_lane=True)


@pytest.mark.parametrize("seed", range(4))
def test_fused_stripe_in_destination_order_equals_oracle(fl, seed):
    core, torch = fl
    rng = np.random.default_rng(400 + seed)
    lanes = int(rng.integers(1, 17))
    chunk = int(rng.choice([8192, 65536, 163840]))
    n = int(rng.integers(1, 700))
    total = n * chunk - int(rng.integers(0, chunk))
    credits = rng.integers(0, 9, size=lanes).astype(np.uint32)
    if seed == 0:
        credits[:] = 0
    epoch_bytes = int(rng.integers(0, 50)) * chunk
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["epoch_bytes"] = epoch_bytes
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                         mode=1, state=st)
    lane_bytes = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    src_np = rng.integers(0, 256, size=total, dtype=np.uint8)
    exp_w = ob.cpu_stripe(src_np, exp_t, lane_bytes)
    src = _dev(torch, src_np)
    wins = [torch.zeros(max(b, 1), dtype=torch.uint8, device="cuda") for b in lane_bytes]
    w = core.make_windows([t.data_ptr() for t in wins], lane_bytes)
    u = core.uniform_params(total, chunk, credits.tolist(), epoch_bytes=epoch_bytes)
    out = core.new_schedule_buffers(n)
    status = core.new_status()
    core.tune("stripe_dest_order", 1)
    try:
        core.stripe_uniform(src, w, u, status, out=out)
        torch.cuda.synchronize()
    finally:
        core.tune("stripe_dest_order", -1)
    assert int(status.item()) == 0
    got_t, got_h = out.table_numpy(), out.hdr_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f"table field {f}")
    np.testing.assert_array_equal(got_h["lane_bytes"], exp_h["lane_bytes"])
    for l in range(lanes):
        np.testing.assert_array_equal(wins[l][: lane_bytes[l]].cpu().numpy(), exp_w[l][: lane_bytes[l]])


def test_schedule_state_carry_and_modes(fl):
    rng = np.random.default_rng(7)
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["epoch_bytes"] = 123456
    st["chunk_index"] = 37
    st["lane_off"][:] = rng.integers(0, 1 << 40, size=16)
    sizes = rng.integers(1, 100000, size=900).astype(np.uint32)
    credits = rng.integers(1, 5, size=(3, 5)).astype(np.uint32)
    for mode in (0, ob.SCHED_RESET_OFFSETS, ob.SCHED_MIRROR):
        _check_schedule(fl, n_lanes=5, credits=credits, quantum=65536, sizes=sizes, epoch_len=50, state=st, mode=mode,
                        src_base=4096)
    src_off = np.cumsum(rng.integers(100000, 200000, size=900)).astype(np.uint64)
    _check_schedule(fl, n_lanes=5, credits=credits, quantum=65536, sizes=sizes, epoch_len=50, src_off=src_off)


def test_schedule_equal_credits_is_static_policy(fl):
    # the reference's live policy: lane = index mod lanes (src/fuselink.h:235)
    core, torch = fl
    sched, _, _ = _check_schedule(fl, n_lanes=8, credits=np.ones(8), quantum=262144, total_bytes=64 << 20,
                                  chunk_bytes=262144)
    t = sched.table_numpy()
    np.testing.assert_array_equal(t["lane"], np.arange(256) % 8)


def _roundtrip(fl, src_np, *, n_lanes, credits, quantum, sizes=None, chunk_bytes=0, epoch_len=0, tile_bytes=32768,
               src_off=None, dst_extra=0):
    core, torch = fl
    nbytes = src_np.size
    sched, exp_t, exp_h = _check_schedule(fl, n_lanes=n_lanes, credits=credits, quantum=quantum, sizes=sizes,
                                          total_bytes=0 if sizes is not None else nbytes, chunk_bytes=chunk_bytes,
                                          epoch_len=epoch_len, tile_bytes=tile_bytes, src_off=src_off)
    caps = [int(b) for b in exp_h["lane_bytes"][:n_lanes]]
    src = _dev(torch, src_np)
    wins = [torch.zeros(max(c, 1) + 64, dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    core.stripe(src, w, sched, status)
    dst = torch.zeros(nbytes + dst_extra, dtype=torch.uint8, device="cuda")
    core.reassemble(dst, w, sched, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    # staged windows equal the host-memcpy windows byte for byte, guard bytes untouched
    exp_w = ob.cpu_stripe(src_np, exp_t, caps)
    for l in range(n_lanes):
        got = wins[l].cpu().numpy()
        np.testing.assert_array_equal(got[: caps[l]], exp_w[l][: caps[l]], err_msg=f"window {l}")
        assert not got[caps[l]:].any(), f"window {l} written past its {caps[l]} bytes"
    exp_dst = ob.cpu_reassemble(nbytes, exp_w, exp_t)
    got_dst = dst.cpu().numpy()
    np.testing.assert_array_equal(got_dst[:nbytes], exp_dst)
    return got_dst


def test_roundtrip_cfg1_shape(fl):
    # 4 MiB uint8, 512 KiB chunks, 2 lanes, equal credits (the reference's operating point)
    rng = np.random.default_rng(1)
    src = rng.integers(0, 256, size=4 << 20, dtype=np.uint8)
    out = _roundtrip(fl, src, n_lanes=2, credits=[1, 1], quantum=512 << 10, chunk_bytes=512 << 10)
    np.testing.assert_array_equal(out, src)


def test_roundtrip_cfg2_shape(fl):
    # 64 MiB fp16 N(0,1), 256 KiB chunks, 8 lanes, credits uniform in [1,8]
    rng = np.random.default_rng(2)
    src = rng.standard_normal(32 << 20, dtype=np.float32).astype(np.float16).view(np.uint8)
    credits = rng.integers(1, 9, size=8)
    out = _roundtrip(fl, src, n_lanes=8, credits=credits, quantum=256 << 10, chunk_bytes=256 << 10)
    np.testing.assert_array_equal(out, src)


@pytest.mark.parametrize("nbytes,chunk", [(1, 4096), (15, 4096), (4097, 4096), ((4 << 20) + 1, 512 << 10),
                                          (1000003, 65536), (3 * 32768, 32768)])
def test_roundtrip_ragged(fl, nbytes, chunk):
    rng = np.random.default_rng(nbytes)
    src = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
    out = _roundtrip(fl, src, n_lanes=3, credits=[2, 1, 3], quantum=chunk, chunk_bytes=chunk)
    np.testing.assert_array_equal(out, src)


def test_roundtrip_odd_sizes_misaligned_windows(fl):
    # chunk sizes that are not multiples of 16 leave window offsets misaligned against the source
    rng = np.random.default_rng(11)
    sizes = rng.integers(1, 70000, size=300).astype(np.uint32)
    src = rng.integers(0, 256, size=int(sizes.sum()), dtype=np.uint8)
    out = _roundtrip(fl, src, n_lanes=4, credits=[1, 2, 3, 4], quantum=32768, sizes=sizes, tile_bytes=4096)
    np.testing.assert_array_equal(out, src)


@pytest.mark.parametrize("tile", [4096, 32768])
def test_every_pair_of_misalignments_and_the_edges_of_the_vector_loop(fl, tile):
    """Source and window misaligned against each other in every combination of the two residues mod 16, with copy
    lengths around everything the shifted copy treats specially: fewer bytes than a vector, a head only, whole
    wavefronts of vectors +- 1 (the last lane takes its second source vector by a load of its own), the unrolled
    block +- 1, a tile +- 1.  One lane, so the window offsets are the running sum of the sizes; explicit source offsets
    choose the source residue.  Windows and reassembled buffer against the oracle's host memcpy."""
    rng = np.random.default_rng(1600 + tile)
    edge = [1, 2, 15, 16, 17, 31, 32, 33, 63 * 16, 64 * 16, 64 * 16 + 5, 65 * 16 + 9, 255 * 16 + 1, 256 * 16, 257 * 16 + 3,
            2047 * 16 + 7, 2048 * 16, 2048 * 16 + 1, 2049 * 16 + 15, tile - 1, tile, tile + 1, 3 * tile + 11]
    sizes, src_off, at = [], [], 0
    for sres in range(16):
        for dres in range(16):
            n = int(edge[(sres * 16 + dres) % len(edge)]) if rng.random() < 0.7 else int(rng.integers(1, 70000))
            # the window stands at residue (sum of the sizes so far) mod 16; steer it to dres with a small filler chunk
            filler = (dres - sum(sizes)) % 16
            if filler:
                sizes.append(filler)
                src_off.append(at)
                at += filler + 16
            at = (at + 15) // 16 * 16 + sres          # the chunk's bytes start at residue sres in the user buffer
            sizes.append(n)
            src_off.append(at)
            at += n + 3
    src = rng.integers(0, 256, size=at + 64, dtype=np.uint8)
    _roundtrip(fl, src, n_lanes=1, credits=[1], quantum=32768, sizes=np.array(sizes, dtype=np.uint32), tile_bytes=tile,
               src_off=np.array(src_off, dtype=np.uint64))


def test_empty_message(fl):
    core, torch = fl
    sched, _, exp_h = _check_schedule(fl, n_lanes=4, credits=[1, 1, 1, 1], quantum=4096, total_bytes=0, chunk_bytes=4096)
    assert exp_h["total_tiles"] == 0
    w = core.make_windows([0, 0, 0, 0], [0, 0, 0, 0])
    status = core.new_status()
    dummy = torch.zeros(1, dtype=torch.uint8, device="cuda")
    core.stripe(dummy[:0], w, sched, status)
    core.reassemble(dummy[:0], w, sched, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0


def test_window_overflow_is_refused_not_written(fl):
    core, torch = fl
    rng = np.random.default_rng(5)
    src_np = rng.integers(0, 256, size=1 << 20, dtype=np.uint8)
    sched, exp_t, exp_h = _check_schedule(fl, n_lanes=2, credits=[1, 1], quantum=65536, total_bytes=1 << 20, chunk_bytes=65536)
    caps = [int(exp_h["lane_bytes"][0]), int(exp_h["lane_bytes"][1]) - 65536]  # lane 1 is one chunk short
    wins = [torch.zeros(int(exp_h["lane_bytes"][l]), dtype=torch.uint8, device="cuda") for l in range(2)]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    core.stripe(_dev(torch, src_np), w, sched, status)
    torch.cuda.synchronize()
    assert int(status.item()) == -5
    assert not wins[1][caps[1]:].cpu().numpy().any()


def test_roundtrip_many_small_chunks_three_search_rounds(fl):
    # > 4096 variable-size chunks: the tile -> row search needs three 64-ary rounds
    rng = np.random.default_rng(13)
    sizes = (rng.integers(0, 200, size=5000) * 16).astype(np.uint32)
    src = rng.integers(0, 256, size=int(sizes.sum()), dtype=np.uint8)
    out = _roundtrip(fl, src, n_lanes=16, credits=rng.integers(0, 4, size=16) + np.eye(16, dtype=np.int64)[3],
                     quantum=1024, sizes=sizes, tile_bytes=1024)
    np.testing.assert_array_equal(out, src)


def test_host_hint_matches_device_header(fl):
    core, torch = fl
    for total, chunk, tile in [(64 << 20, 256 << 10, 32768), ((4 << 20) + 1, 512 << 10, 32768), (5, 4096, 4096), (0, 4096, 4096)]:
        sched, _, exp_h = _check_schedule(fl, n_lanes=4, credits=[1, 2, 3, 4], quantum=chunk, total_bytes=total,
                                          chunk_bytes=chunk, tile_bytes=tile)
        h = core.uniform_hint(total, chunk, tile)
        assert (h.total_tiles, h.n_chunks, h.uniform_tiles) == (exp_h["total_tiles"], exp_h["n_chunks"], exp_h["uniform_tiles"])


def test_roundtrip_with_host_hint(fl):
    core, torch = fl
    rng = np.random.default_rng(21)
    nbytes, chunk = (8 << 20) + 4096 + 7, 256 << 10
    src_np = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
    sched, exp_t, exp_h = _check_schedule(fl, n_lanes=8, credits=rng.integers(1, 9, size=8), quantum=chunk,
                                          total_bytes=nbytes, chunk_bytes=chunk)
    caps = [int(b) for b in exp_h["lane_bytes"][:8]]
    wins = [torch.zeros(max(c, 1), dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    hint = core.uniform_hint(nbytes, chunk)
    src = _dev(torch, src_np)
    dst = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    core.stripe(src, w, sched, status, hint=hint)
    core.reassemble(dst, w, sched, status, hint=hint)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    np.testing.assert_array_equal(dst.cpu().numpy(), src_np)
    exp_w = ob.cpu_stripe(src_np, exp_t, caps)
    for l in range(8):
        np.testing.assert_array_equal(wins[l].cpu().numpy()[: caps[l]], exp_w[l][: caps[l]])


@pytest.mark.parametrize("fast", [1, 0])
@pytest.mark.parametrize("seed", range(8))
def test_schedule_uniform_closed_form_and_scan_agree_with_oracle(fl, seed, fast):
    """Quantum-sized chunks take the closed-form kernel (fast=1) or are forced through the scan
    kernel (fast=0); both must equal the oracle, with epochs, empty credit rows, carried state and
    every mode bit in play."""
    core, torch = fl
    core.tune("sched_uniform_fast", fast)
    try:
        rng = np.random.default_rng(1000 + seed)
        lanes = int(rng.integers(1, 17))
        rows = int(rng.integers(1, 33))
        chunk = int(rng.choice([128, 4096, 65536, 100 * 128]))
        n = int(rng.choice([1, 2, 255, 256, 257, 1000, 3000]))
        total = n * chunk - int(rng.integers(0, chunk))
        credits = rng.integers(0, 9, size=(rows, lanes)).astype(np.uint32)
        credits[rng.integers(0, rows)] = 0
        epoch_len = int(rng.choice([0, 1, 8, 100, 1000]))
        st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
        st["chunk_index"] = int(rng.integers(0, 5000))
        st["epoch_bytes"] = int(rng.integers(0, 50)) * chunk + int(rng.integers(0, chunk))
        st["lane_off"][:] = rng.integers(0, 1 << 36, size=16)
        for mode in (0, ob.SCHED_RESET_OFFSETS, ob.SCHED_MIRROR, 4, 5):
            _check_schedule(fl, n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                            epoch_len=epoch_len, state=st, mode=mode, src_base=int(rng.integers(0, 1 << 20)),
                            tile_bytes=int(rng.choice([128, 4096, 32768, 3 * 128])))
        _check_schedule(fl, n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk, epoch_len=epoch_len)
    finally:
        core.tune("sched_uniform_fast", 1)


def test_schedule_chain_of_calls_matches_one_shot(fl):
    # a message scheduled in pieces with the device-resident state equals the one-shot table
    core, torch = fl
    rng = np.random.default_rng(77)
    chunk, lanes, E = 4096, 5, 37
    credits = rng.integers(0, 5, size=(3, lanes)).astype(np.uint32)
    pieces = [10 * chunk, 600 * chunk, chunk, 300 * chunk + 5]
    whole_t, _, whole_s = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=sum(pieces),
                                             chunk_bytes=chunk, epoch_len=E)
    d_credits = _dev(torch, credits.view(np.int32))
    state = core.new_state()
    got, base = [], 0
    for nb in pieces:
        sched = core.schedule(n_lanes=lanes, credits=d_credits, quantum=chunk, total_bytes=nb, chunk_bytes=chunk, epoch_len=E,
                              state=state, src_base=base)
        torch.cuda.synchronize()
        got.append(sched.table_numpy())
        base += nb
    cat = np.concatenate(got)
    for f in ("src_off", "win_off", "len", "lane", "epoch"):
        np.testing.assert_array_equal(cat[f], whole_t[f], err_msg=f)
    s = core.state_numpy(state)
    assert s["chunk_index"] == whole_s["chunk_index"] and (s["lane_off"] == whole_s["lane_off"]).all()


@pytest.mark.parametrize("fast", [1, 0])
@pytest.mark.parametrize("seed", range(7))
def test_fused_schedule_and_stripe_equals_oracle(fl, seed, fast):
    """flh_stripe_uniform / flh_reassemble_uniform: the table it writes, the staged windows and the
    reassembled buffer against the oracle, with carried epoch bytes and an empty credit row; with the
    host-prepared reciprocal (fast=1), with in-kernel division (fast=0), and with a credit row that
    sums past 32 bits (seed 6), which must fall back to division by itself."""
    core, torch = fl
    core.tune("fused_fast", fast)
    try:
        _fused_case(fl, seed)
    finally:
        core.tune("fused_fast", 1)


def _fused_case(fl, seed):
    core, torch = fl
    rng = np.random.default_rng(500 + seed)
    lanes = int(rng.integers(1, 17))
    chunk = int(rng.choice([4096, 65536, 256 << 10, 100 * 128]))
    n = int(rng.choice([1, 2, 7, 64, 257]))
    total = n * chunk - int(rng.integers(0, chunk))
    tile = int(rng.choice([4096, 32768, 3 * 128]))
    credits = rng.integers(0, 9, size=lanes).astype(np.uint32)
    if seed == 3:
        credits[:] = 0
    if seed == 6:
        credits = rng.integers(2**31, 2**32 - 1, size=lanes).astype(np.uint32)
        credits[0] = 3
    epoch_bytes = int(rng.integers(0, 40)) * chunk + int(rng.integers(0, chunk))
    base = int(rng.integers(0, 8)) * 4096
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["epoch_bytes"] = epoch_bytes
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                         tile_bytes=tile, mode=ob.SCHED_RESET_OFFSETS, state=st, src_base=base)
    src_np = rng.integers(0, 256, size=base + total, dtype=np.uint8)
    src = _dev(torch, src_np)
    caps = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    wins = [torch.zeros(max(c, 1) + 64, dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    u = core.uniform_params(total, chunk, credits, src_base=base, epoch_bytes=epoch_bytes, tile_bytes=tile)
    out = core.new_schedule_buffers(n, tile)
    core.stripe_uniform(src, w, u, status, out=out)
    dst = torch.zeros_like(src)
    core.reassemble_uniform(dst, w, u, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    got_t, got_h = out.table_numpy(), out.hdr_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f)
    for f in ("total_bytes", "total_tiles", "n_chunks", "flags", "uniform_tiles", "lane_bytes", "lane_chunks"):
        np.testing.assert_array_equal(got_h[f], exp_h[f], err_msg=f)
    exp_w = ob.cpu_stripe(src_np, exp_t, caps)
    for l in range(lanes):
        got = wins[l].cpu().numpy()
        np.testing.assert_array_equal(got[: caps[l]], exp_w[l][: caps[l]])
        assert not got[caps[l]:].any()
    got_dst = dst.cpu().numpy()
    np.testing.assert_array_equal(got_dst[base:], src_np[base:])
    assert not got_dst[:base].any()
    # the unfused path produces the same windows from the same table
    sched = core.schedule(n_lanes=lanes, credits=[int(c) for c in credits], quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                          tile_bytes=tile, mode=core.SCHED_RESET_OFFSETS, src_base=base,
                          state=_dev(torch, np.array([st], dtype=ob.STATE_DTYPE).view(np.uint8)))
    torch.cuda.synchronize()
    assert sched.table_numpy().tobytes() == got_t.tobytes()


def test_fused_refuses_short_window(fl):
    core, torch = fl
    src = torch.randint(0, 255, (1 << 20,), dtype=torch.uint8, device="cuda")
    wins = [torch.zeros(512 << 10, dtype=torch.uint8, device="cuda") for _ in range(2)]
    w = core.make_windows([t.data_ptr() for t in wins], [512 << 10, (512 << 10) - 65536])
    status = core.new_status()
    core.stripe_uniform(src, w, core.uniform_params(1 << 20, 65536, [1, 1]), status)
    torch.cuda.synchronize()
    assert int(status.item()) == -5


@pytest.mark.parametrize("seed", range(6))
def test_batch_of_requests_is_one_message(fl, seed):
    """flh_stripe_batch / flh_reassemble_batch: several request buffers scheduled and copied as the
    concatenation they form.  Table, header and staged windows equal the oracle's for the single
    message; every destination receives its own source."""
    core, torch = fl
    rng = np.random.default_rng(700 + seed)
    lanes = int(rng.integers(1, 17))
    chunk = int(rng.choice([4096, 65536, 512 << 10, 100 * 128]))
    n_req = int(rng.integers(1, 9))
    sizes = [int(rng.integers(1, 6)) * chunk for _ in range(n_req)]
    sizes[-1] -= int(rng.integers(0, chunk))            # only the last request may end inside a chunk
    total = sum(sizes)
    credits = rng.integers(0, 9, size=lanes).astype(np.uint32)
    if seed == 2:
        credits[:] = 0
    epoch_bytes = int(rng.integers(0, 40)) * chunk
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["epoch_bytes"] = epoch_bytes
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                         mode=ob.SCHED_RESET_OFFSETS, state=st)
    srcs_np = [rng.integers(0, 256, size=s, dtype=np.uint8) for s in sizes]
    caps = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    exp_w = ob.cpu_stripe(np.concatenate(srcs_np), exp_t, caps)
    srcs = [_dev(torch, a) for a in srcs_np]
    dsts = [torch.zeros(s + 64, dtype=torch.uint8, device="cuda") for s in sizes]
    wins = [torch.zeros(max(c, 1) + 64, dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    b = core.batch_params(srcs, dsts, chunk, credits.tolist(), epoch_bytes=epoch_bytes)
    out = core.new_schedule_buffers(len(exp_t))
    core.stripe_batch(b, w, status, out=out)
    core.reassemble_batch(b, w, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    got_t, got_h = out.table_numpy(), out.hdr_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f)
    for f in ("total_bytes", "total_tiles", "n_chunks", "flags", "lane_bytes", "lane_chunks"):
        np.testing.assert_array_equal(got_h[f], exp_h[f], err_msg=f)
    for l in range(lanes):
        got = wins[l].cpu().numpy()
        np.testing.assert_array_equal(got[: caps[l]], exp_w[l][: caps[l]])
        assert not got[caps[l]:].any()
    for q in range(n_req):
        got = dsts[q].cpu().numpy()
        np.testing.assert_array_equal(got[: sizes[q]], srcs_np[q])
        assert not got[sizes[q]:].any()


@pytest.mark.parametrize("seed", range(8))
def test_batch_of_segments_equals_the_oracle_segment_by_segment(fl, seed):
    """flh_stripe_batch / flh_reassemble_batch with several segments: each segment is scheduled as the message its requests
    form, from its own epoch prefix under its own credit row, and the segments follow each other in the windows at 128-byte
    boundaries.  Rows, header, flh_batch_layout, the staged bytes and every destination against the oracle."""
    core, torch = fl
    rng = np.random.default_rng(8800 + seed)
    lanes = int(rng.integers(1, 17))
    chunk = int(rng.choice([4096, 65536, 256 << 10, 100 * 128]))
    n_seg = int(rng.integers(1, 9))
    segments, sizes = [], []
    for k in range(n_seg):
        room = 32 - len(sizes) - (n_seg - 1 - k)
        n_req = int(rng.integers(1, max(2, min(6, room + 1))))
        ss = [int(rng.integers(1, 4)) * chunk for _ in range(n_req)]
        if rng.random() < 0.6:
            ss[-1] -= int(rng.integers(1, chunk))            # a segment's last request may end inside a chunk
        credits = rng.integers(0, 9, size=lanes).astype(np.uint32)
        if seed == 3 and k == 0:
            credits[:] = 0                                   # no credit anywhere: the static policy stands in
        segments.append((n_req, credits, int(rng.integers(0, 50)) * chunk))
        sizes += ss
    srcs_np = [rng.integers(0, 256, size=s, dtype=np.uint8) for s in sizes]
    srcs = [_dev(torch, a) for a in srcs_np]
    dsts = [torch.zeros(s + 64, dtype=torch.uint8, device="cuda") for s in sizes]
    b = core.batch_params(srcs, dsts, chunk, [1] * lanes, segments=[(n, c.tolist(), e) for n, c, e in segments])
    # the oracle, segment by segment; windows as the layout rule says
    lane_end = np.zeros(16, dtype=np.uint64)
    exp_rows, exp_bases, staged = [], [], {}
    lane_bytes_sum, lane_chunks_sum, flags, first_row, q = np.zeros(16, np.uint64), np.zeros(16, np.uint32), 0, 0, 0
    tiles_per_chunk = (chunk + 32767) // 32768
    total_tiles = 0
    for n_req, credits, epoch in segments:
        seg_np = np.concatenate(srcs_np[q:q + n_req])
        q += n_req
        st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
        st["epoch_bytes"] = epoch
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=seg_np.size, chunk_bytes=chunk,
                                             mode=ob.SCHED_RESET_OFFSETS, state=st)
        base = (lane_end + np.uint64(127)) // np.uint64(128) * np.uint64(128)
        exp_bases.append(base.copy())
        wins_seg = ob.cpu_stripe(seg_np, exp_t, [int(x) for x in exp_h["lane_bytes"][:lanes]])
        for l in range(lanes):
            n = int(exp_h["lane_bytes"][l])
            if n:
                staged[(len(exp_rows), l)] = (int(base[l]), wins_seg[l][:n])
        rows = exp_t.copy()
        rows["win_off"] += base[rows["lane"]]
        rows["tile_base"] += first_row * tiles_per_chunk
        exp_rows.append(rows)
        used = exp_h["lane_chunks"] > 0
        lane_end[used] = base[used] + exp_h["lane_bytes"][used]
        lane_bytes_sum += exp_h["lane_bytes"]
        lane_chunks_sum += exp_h["lane_chunks"]
        flags |= int(exp_h["flags"])
        total_tiles += int(exp_h["total_tiles"])
        first_row += len(exp_t)
    exp_t = np.concatenate(exp_rows)
    ends, bases = core.batch_layout(b)
    np.testing.assert_array_equal(np.array(ends, dtype=np.uint64), lane_end)
    for k in range(n_seg):
        np.testing.assert_array_equal(np.array(bases[k], dtype=np.uint64), exp_bases[k], err_msg=f"segment {k} bases")
    caps = [int(x) for x in lane_end[:lanes]]
    wins = [torch.zeros(max(c, 1) + 64, dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    status = core.new_status()
    out = core.new_schedule_buffers(len(exp_t))
    core.stripe_batch(b, w, status, out=out)
    core.reassemble_batch(b, w, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    got_t, got_h = out.table_numpy(), out.hdr_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f)
    np.testing.assert_array_equal(got_h["lane_bytes"], lane_bytes_sum)
    np.testing.assert_array_equal(got_h["lane_chunks"], lane_chunks_sum)
    assert int(got_h["total_bytes"]) == sum(sizes) and int(got_h["n_chunks"]) == len(exp_t)
    assert int(got_h["flags"]) == flags and int(got_h["total_tiles"]) == total_tiles
    for (k, l), (off, data) in staged.items():
        np.testing.assert_array_equal(wins[l].cpu().numpy()[off:off + data.size], data, err_msg=f"segment {k} lane {l}")
    for i, s in enumerate(sizes):
        got = dsts[i].cpu().numpy()
        np.testing.assert_array_equal(got[:s], srcs_np[i])
        assert not got[s:].any()


def test_batch_refuses_segments_that_do_not_add_up(fl):
    core, torch = fl
    chunk = 4096
    srcs = [torch.zeros(chunk, dtype=torch.uint8, device="cuda") for _ in range(3)]
    dsts = [torch.zeros_like(t) for t in srcs]
    wins = [torch.zeros(8 * chunk, dtype=torch.uint8, device="cuda") for _ in range(2)]
    w = core.make_windows([t.data_ptr() for t in wins], [8 * chunk] * 2)
    b = core.batch_params(srcs, dsts, chunk, [1, 1], segments=[(1, [1, 1], 0), (1, [1, 0], 0)])
    with pytest.raises(Exception, match="segments hold 2 requests"):
        core.stripe_batch(b, w, core.new_status())
    b = core.batch_params(srcs, dsts, chunk, [1, 1], segments=[(2, [1, 1], 0), (2, [1, 0], 0)])
    with pytest.raises(Exception, match="are left"):
        core.stripe_batch(b, w, core.new_status())


def test_batch_refuses_a_request_that_ends_inside_a_chunk(fl):
    core, torch = fl
    chunk = 4096
    srcs = [torch.zeros(chunk + 1, dtype=torch.uint8, device="cuda"), torch.zeros(chunk, dtype=torch.uint8, device="cuda")]
    dsts = [torch.zeros_like(t) for t in srcs]
    wins = [torch.zeros(4 * chunk, dtype=torch.uint8, device="cuda") for _ in range(2)]
    w = core.make_windows([t.data_ptr() for t in wins], [4 * chunk] * 2)
    b = core.batch_params(srcs, dsts, chunk, [1, 1])
    with pytest.raises(Exception, match="whole number of chunks"):
        core.stripe_batch(b, w, core.new_status())


@pytest.mark.parametrize("mode_out,mode_in", [(0, 0), (1, 2), (3, 3), (2, 1)])
def test_forced_streaming_modes_move_the_same_bytes(fl, mode_out, mode_in):
    """The cache policy of a launch (which side streams past the caches) selects another instantiation of
    the copy kernels; every one of them must leave the same windows and the same reassembled buffer."""
    core, torch = fl
    rng = np.random.default_rng(9100 + 4 * mode_out + mode_in)
    lanes, chunk = 6, 40960
    total = 333 * chunk - 777
    credits = rng.integers(0, 7, size=lanes).astype(np.uint32)
    credits[2] = 3
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk)
    lane_bytes = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    src_np = rng.integers(0, 256, size=total, dtype=np.uint8)
    exp_w = ob.cpu_stripe(src_np, exp_t, lane_bytes)
    src = _dev(torch, src_np)
    core.tune("stream_mode_out", mode_out)
    core.tune("stream_mode_in", mode_in)
    try:
        for fused in (False, True):
            wins = [torch.zeros(max(b, 1), dtype=torch.uint8, device="cuda") for b in lane_bytes]
            w = core.make_windows([t.data_ptr() for t in wins], lane_bytes)
            status = core.new_status()
            dst = torch.zeros_like(src)
            if fused:
                u = core.uniform_params(total, chunk, credits.tolist())
                out = core.new_schedule_buffers(len(exp_t))
                core.stripe_uniform(src, w, u, status, out=out)
                core.reassemble_uniform(dst, w, u, status)
            else:
                sched = core.schedule(n_lanes=lanes, credits=credits.tolist(), quantum=chunk, total_bytes=total, chunk_bytes=chunk)
                core.stripe(src, w, sched, status)
                core.reassemble(dst, w, sched, status)
            torch.cuda.synchronize()
            assert int(status.item()) == 0
            for l in range(lanes):
                if lane_bytes[l]:
                    np.testing.assert_array_equal(wins[l].cpu().numpy()[:lane_bytes[l]], exp_w[l][:lane_bytes[l]], err_msg=f"lane {l}")
            assert torch.equal(src, dst)
    finally:
        core.tune("stream_mode_out", -1)
        core.tune("stream_mode_in", -1)


def test_launches_record_into_a_hip_graph_and_replay(fl):
    """No entry point on the data path allocates, clears or synchronizes, so a caller may record
    schedule -> stripe -> reassemble into a HIP graph, and likewise the launch that stages and delivers and the
    one that stages and carries.  Every replay, with eager work and synchronizations of the program's own in between,
    must give what the eager launches give for the source bytes of that moment."""
    core, torch = fl
    rng = np.random.default_rng(31337)
    lanes, chunk = 8, 65536
    total = 300 * chunk - 4097
    credits = rng.integers(1, 9, size=lanes).astype(np.uint32)
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk)
    lane_bytes = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    src = torch.zeros(total, dtype=torch.uint8, device="cuda")
    dst_fused, dst_table, dst_deliver = torch.zeros_like(src), torch.zeros_like(src), torch.zeros_like(src)
    wins = [torch.zeros(max(b, 1), dtype=torch.uint8, device="cuda") for b in lane_bytes]
    w = core.make_windows([t.data_ptr() for t in wins], lane_bytes)
    wins2 = [torch.zeros(max(b, 1), dtype=torch.uint8, device="cuda") for b in lane_bytes]
    land = [torch.zeros(max(b, 1), dtype=torch.uint8, device="cuda") for b in lane_bytes]
    w2 = core.make_windows([t.data_ptr() for t in wins2], lane_bytes)
    wl = core.make_windows([t.data_ptr() for t in land], lane_bytes)
    u = core.uniform_params(total, chunk, credits.tolist())
    out = core.new_schedule_buffers(len(exp_t))
    sched_out = core.new_schedule_buffers(len(exp_t))
    d_credits = _dev(torch, credits.view(np.int32))
    status = core.new_status()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        # fused pair, then the three-launch path over the same windows into a second destination
        core.stripe_uniform(src, w, u, status, out=out)
        core.reassemble_uniform(dst_fused, w, u, status)
        sched = core.schedule(n_lanes=lanes, credits=d_credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk, out=sched_out)
        core.stripe(src, w, sched, status)
        core.reassemble(dst_table, w, sched, status)
        # one launch that stages and delivers; one that stages and carries into landing windows
        core.stage_deliver_uniform(src, dst_deliver, w2, u, status)
        core.stripe_uniform_carry(src, w2, wl, u, status)
    for rep in range(4):
        src_np = rng.integers(0, 256, size=total, dtype=np.uint8)
        src.copy_(torch.from_numpy(src_np))
        dst_fused.zero_()
        dst_table.zero_()
        dst_deliver.zero_()
        for t in wins + wins2 + land:
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(status.item()) == 0
        assert torch.equal(dst_fused, src) and torch.equal(dst_table, src) and torch.equal(dst_deliver, src), f"replay {rep}"
        exp_w = ob.cpu_stripe(src_np, exp_t, lane_bytes)
        for l in range(lanes):
            for name, ws in (("windows", wins), ("windows of the delivering launch", wins2), ("landing windows", land)):
                np.testing.assert_array_equal(ws[l].cpu().numpy()[:lane_bytes[l]], exp_w[l][:lane_bytes[l]], err_msg=f"replay {rep} {name} lane {l}")
        for f in ob.DESC_DTYPE.names:
            np.testing.assert_array_equal(out.table_numpy()[f], exp_t[f], err_msg=f"replay {rep} field {f}")
            np.testing.assert_array_equal(sched_out.table_numpy()[f], exp_t[f], err_msg=f"replay {rep} field {f} (scheduler kernel)")


def test_fused_launch_at_and_past_its_chunk_limit(fl):
    """One fused launch names its chunks through the grid's second dimension: 65 535 of them are taken (and come
    out as the oracle has them), one more is refused with an error before anything is launched."""
    core, torch = fl
    rng = np.random.default_rng(65535)
    lanes, chunk = 5, 256
    credits = np.array([3, 1, 0, 2, 2], dtype=np.uint32)
    for n, ok in ((65535, True), (65536, False)):
        total = n * chunk - 100
        src_np = rng.integers(0, 256, size=total, dtype=np.uint8)
        src = _dev(torch, src_np)
        dst = torch.zeros_like(src)
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                             tile_bytes=256)
        lane_bytes = [int(b) for b in exp_h["lane_bytes"][:lanes]]
        wins = [torch.zeros(max(b, 1), dtype=torch.uint8, device="cuda") for b in lane_bytes]
        w = core.make_windows([t.data_ptr() for t in wins], lane_bytes)
        u = core.uniform_params(total, chunk, credits.tolist(), tile_bytes=256)
        out = core.new_schedule_buffers(n, tile_bytes=256)
        status = core.new_status()
        if not ok:
            with pytest.raises(Exception, match="65535"):
                core.stripe_uniform(src, w, u, status, out=out)
            continue
        core.stripe_uniform(src, w, u, status, out=out)
        core.reassemble_uniform(dst, w, u, status)
        torch.cuda.synchronize()
        assert int(status.item()) == 0 and torch.equal(src, dst)
        got_t = out.table_numpy()
        for f in ob.DESC_DTYPE.names:
            np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f"table field {f}")
        exp_w = ob.cpu_stripe(src_np, exp_t, lane_bytes)
        for l in range(lanes):
            if lane_bytes[l]:
                np.testing.assert_array_equal(wins[l].cpu().numpy()[:lane_bytes[l]], exp_w[l][:lane_bytes[l]], err_msg=f"lane {l}")


@pytest.mark.parametrize("lanes,hot", [(1, 0), (8, 2), (16, 15)])
def test_fused_pair_with_one_lane_named_outright(fl, lanes, hot):
    """The static policy (lane = channelId % nNics, FuseLink src/fuselink.h:235) reaches the kernels as a credit row
    with a single 1: every chunk on that lane, window offsets running, other windows untouched."""
    core, torch = fl
    rng = np.random.default_rng(1235 + lanes)
    chunk = 24576
    total = 77 * chunk - 5
    credits = np.zeros(lanes, dtype=np.uint32)
    credits[hot] = 1
    epoch_bytes = 9 * chunk
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["epoch_bytes"] = epoch_bytes
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                         mode=1, state=st)
    assert (exp_t["lane"] == hot).all()
    src_np = rng.integers(0, 256, size=total, dtype=np.uint8)
    src = _dev(torch, src_np)
    dst = torch.zeros_like(src)
    wins = [torch.full((total + 64,), 0xA5, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
    w = core.make_windows([t.data_ptr() for t in wins], [total] * lanes)
    u = core.uniform_params(total, chunk, credits.tolist(), epoch_bytes=epoch_bytes)
    out = core.new_schedule_buffers(len(exp_t))
    status = core.new_status()
    core.stripe_uniform(src, w, u, status, out=out)
    core.reassemble_uniform(dst, w, u, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and torch.equal(src, dst)
    got_t = out.table_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f"table field {f}")
    for l in range(lanes):
        got = wins[l].cpu().numpy()
        if l == hot:
            np.testing.assert_array_equal(got[:total], src_np)
            assert (got[total:] == 0xA5).all()
        else:
            assert (got == 0xA5).all(), f"lane {l} was written"


def _expected_tiles(table, tile):
    """One descriptor per copy tile, from the table alone: tile j of row r sits at tile_base[r] + j."""
    rows = []
    for r, d in enumerate(table):
        nt = (int(d["len"]) + tile - 1) // tile
        for j in range(nt):
            off = j * tile
            rows.append((int(d["src_off"]) + off, int(d["win_off"]) + off, min(tile, int(d["len"]) - off), int(d["lane"]), r,
                         int(d["tile_base"]) + j))
    return rows


@pytest.mark.parametrize("seed", range(10))
def test_tile_descriptors_and_the_copies_they_drive_equal_oracle(fl, seed):
    """flh_schedule with d_tiles, then flh_stripe_tiles / flh_reassemble_tiles: descriptors as the table implies them,
    windows and reassembled bytes as the oracle's, for variable sizes (empty chunks among them), explicit source
    offsets with gaps and odd alignment, small and large tiles, with and without the host copy of the header."""
    core, torch = fl
    rng = np.random.default_rng(8800 + seed)
    lanes = int(rng.integers(1, 17))
    tile = int(rng.choice([128, 4096, 32768]))
    n = int(rng.integers(1, 1200))
    sizes = rng.integers(0, int(rng.choice([300, 9000, 70000])), size=n).astype(np.uint32)
    if seed % 3 == 0:
        sizes[rng.integers(0, n, size=max(1, n // 7))] = 0
    credits = rng.integers(0, 9, size=(int(rng.integers(1, 4)), lanes)).astype(np.uint32)
    epoch_len = int(rng.choice([0, 5, 100]))
    quantum = int(rng.choice([1, 4096, 65536]))
    src_off = None
    if seed % 2:
        gaps = rng.integers(0, 40, size=n)
        src_off = np.concatenate([[int(rng.integers(0, 64))], (sizes[:-1] + gaps[:-1])]).cumsum().astype(np.uint64)
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=quantum, sizes=sizes, src_off=src_off,
                                         epoch_len=epoch_len, tile_bytes=tile)
    total = int((src_off[-1] + sizes[-1]) if src_off is not None else sizes.sum()) + 8
    n_tiles = int(exp_h["total_tiles"])
    cap = n_tiles + int(rng.integers(0, 50))
    sched = core.schedule(n_lanes=lanes, credits=_dev(torch, credits.view(np.int32)), quantum=quantum, sizes=_dev(torch, sizes.view(np.int32)),
                          src_off=None if src_off is None else _dev(torch, src_off.view(np.int64)), epoch_len=epoch_len, tile_bytes=tile,
                          tiles_capacity=max(cap, 1))
    torch.cuda.synchronize()
    got_t = sched.table_numpy()
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f"table field {f}")
    got = sched.tiles_numpy(n_tiles)
    want = _expected_tiles(exp_t, tile)
    assert len(want) == n_tiles
    for (s_off, w_off, ln, lane, row, t) in want:
        g = got[t]
        assert (int(g["src_off"]), int(g["win_off"]), int(g["len"]), int(g["lane"]), int(g["row"])) == (s_off, w_off, ln, lane, row), f"tile {t}"
    caps = [int(b) for b in exp_h["lane_bytes"][:lanes]]
    src_np = rng.integers(0, 256, size=total, dtype=np.uint8)
    exp_w = ob.cpu_stripe(src_np, exp_t, caps)
    src = _dev(torch, src_np)
    hdr = sched.hdr_numpy()
    hint = core.SchedHdr()
    hint.total_bytes, hint.total_tiles, hint.n_chunks = int(hdr["total_bytes"]), int(hdr["total_tiles"]), int(hdr["n_chunks"])
    for h in (None, hint):
        pad = [int(rng.integers(0, 16)) for _ in caps]      # misaligned window bases
        wins = [torch.zeros(c + 64, dtype=torch.uint8, device="cuda") for c in caps]
        w = core.make_windows([t.data_ptr() + p for t, p in zip(wins, pad)], caps)
        status = core.new_status()
        dst = torch.zeros_like(src)
        core.stripe(src, w, sched, status, hint=h)
        core.reassemble(dst, w, sched, status, hint=h)
        torch.cuda.synchronize()
        assert int(status.item()) == 0
        for l in range(lanes):
            np.testing.assert_array_equal(wins[l].cpu().numpy()[pad[l]: pad[l] + caps[l]], exp_w[l][:caps[l]], err_msg=f"lane {l}")
        exp_dst = ob.cpu_reassemble(total, exp_w, exp_t)
        np.testing.assert_array_equal(dst.cpu().numpy(), exp_dst[:total])


def test_tile_descriptor_array_too_small_is_refused(fl):
    core, torch = fl
    sizes = np.full(40, 70000, dtype=np.uint32)      # 3 tiles each: 120 tiles
    sched = core.schedule(n_lanes=2, credits=[1, 1], quantum=70000, sizes=_dev(torch, sizes.view(np.int32)), tiles_capacity=100)
    src = torch.zeros(40 * 70000, dtype=torch.uint8, device="cuda")
    wins = [torch.zeros(20 * 70000, dtype=torch.uint8, device="cuda") for _ in range(2)]
    w = core.make_windows([t.data_ptr() for t in wins], [20 * 70000] * 2)
    status = core.new_status()
    core.stripe(src, w, sched, status)                # header only on the device: the kernel finds out
    torch.cuda.synchronize()
    assert int(status.item()) == -5                   # FLH_E_RANGE
    hint = core.SchedHdr()
    hint.total_tiles, hint.n_chunks = 120, 40
    with pytest.raises(Exception, match="120 tiles"):
        core.stripe(src, w, sched, status, hint=hint)  # the host copy of the header says so before anything is launched


@pytest.mark.parametrize("seed", range(24))
def test_scan_scheduler_over_several_workgroups_equals_oracle(fl, seed):
    """With a workspace a long list is scheduled by one workgroup per 1024 chunks in three launches; table, header
    and carried state must be the one-workgroup kernel's, i.e. the oracle's: variable and uniform sizes, epochs that
    start inside, at the edge of and nowhere near a segment, several credit rows (a rowless one among them), explicit
    source offsets, carried state from an earlier call, every mode bit."""
    core, torch = fl
    rng = np.random.default_rng(4100 + seed)
    lanes = int(rng.integers(1, 17))
    n = int(rng.choice([1, 700, 1024, 1025, 2048, 3000, 4097, 9000]))
    rows = int(rng.integers(1, 6))
    credits = rng.integers(0, 9, size=(rows, lanes)).astype(np.uint32)
    if seed % 4 == 0 and rows > 1:
        credits[1, :] = 0
    epoch_len = int(rng.choice([0, 7, 512, 1024, 1000, 5000]))
    quantum = int(rng.choice([1, 4096, 65536, 100000]))
    tile = int(rng.choice([128, 4096, 32768]))
    mode = int(rng.choice([0, 1, 2, 4, 5]))
    state = None
    if seed % 2:
        state = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
        state["epoch_bytes"] = int(rng.integers(0, 1 << 22))
        state["chunk_index"] = int(rng.integers(0, 3000))
        state["lane_off"][:lanes] = rng.integers(0, 1 << 30, size=lanes)
    kw = dict(n_lanes=lanes, credits=credits, quantum=quantum, epoch_len=epoch_len, tile_bytes=tile, mode=mode, state=state, workspace=True)
    core.tune("sched_seg_min", 1)
    try:
        if seed % 3 == 2:      # uniform sizes that still need the scan (quantum != chunk)
            chunk = int(rng.choice([4096, 50000]))
            total = n * chunk - int(rng.integers(0, chunk))
            if quantum == chunk:
                kw["quantum"] = chunk + 1
            _check_schedule(fl, total_bytes=total, chunk_bytes=chunk, src_base=int(rng.integers(0, 1 << 20)), **kw)
        else:
            sizes = rng.integers(0, int(rng.choice([300, 9000, 200000])), size=n).astype(np.uint32)
            src_off = None
            if seed % 3 == 1:
                src_off = (np.concatenate([[5], sizes[:-1].astype(np.uint64) + 3]).cumsum()).astype(np.uint64)
            _check_schedule(fl, sizes=sizes, src_off=src_off, **kw)
    finally:
        core.tune("sched_seg_min", 4096)


def test_scan_scheduler_workspace_too_small_is_refused(fl):
    """A workspace that cannot hold the partials of every segment is an argument error, raised before any launch."""
    import ctypes as C

    from fuselink_amd import _lib
    core, torch = fl
    n = 9000
    sizes = _dev(torch, np.full(n, 4096, dtype=np.int32))
    out = core.new_schedule_buffers(n)
    small = torch.zeros(64, dtype=torch.uint8, device="cuda")
    p = _lib.SchedParams(sizes.data_ptr(), 0, 0, None, 0, n, 2, None, 1, 0, 4096, 32768, 0, None, out.table.data_ptr(), out.hdr.data_ptr())
    p.inline_credits[0] = p.inline_credits[1] = 1
    p.d_workspace, p.workspace_bytes = small.data_ptr(), small.numel()
    assert int(_lib.load().flh_schedule_workspace_bytes(n)) > small.numel()
    with pytest.raises(Exception, match="workspace"):
        _lib.check(_lib.load().flh_schedule(C.byref(p), None))


def test_long_variable_list_records_into_a_hip_graph(fl):
    """The scan over several workgroups, the expansion to tile descriptors and the copies that read them are plain
    launches too: recorded once, replayed with new sizes and bytes in the same buffers, checked against the oracle."""
    core, torch = fl
    rng = np.random.default_rng(2718)
    lanes, n, tile = 7, 9000, 4096
    credits = rng.integers(0, 6, size=(3, lanes)).astype(np.uint32)
    cap_bytes = n * 3000
    src = torch.zeros(cap_bytes, dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    sizes = torch.zeros(n, dtype=torch.int32, device="cuda")
    wins = [torch.zeros(cap_bytes, dtype=torch.uint8, device="cuda") for _ in range(lanes)]
    w = core.make_windows([t.data_ptr() for t in wins], [cap_bytes] * lanes)
    d_credits = _dev(torch, credits.view(np.int32))
    status = core.new_status()
    sched = core.new_schedule_buffers(n, tile_bytes=tile)
    tiles_capacity = cap_bytes // tile + n
    # buffers the graph will use must exist before the capture: one eager call allocates workspace and descriptors
    core.schedule(n_lanes=lanes, credits=d_credits, quantum=2048, sizes=sizes, epoch_len=1000, tile_bytes=tile, out=sched,
                  tiles_capacity=tiles_capacity, workspace=True)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        core.schedule(n_lanes=lanes, credits=d_credits, quantum=2048, sizes=sizes, epoch_len=1000, tile_bytes=tile, out=sched,
                      tiles_capacity=tiles_capacity, workspace=True)
        core.stripe(src, w, sched, status)
        core.reassemble(dst, w, sched, status)
    for rep in range(3):
        sizes_np = rng.integers(0, 3000, size=n).astype(np.uint32)
        total = int(sizes_np.sum())
        src_np = rng.integers(0, 256, size=cap_bytes, dtype=np.uint8)
        sizes.copy_(torch.from_numpy(sizes_np.view(np.int32)))
        src.copy_(torch.from_numpy(src_np))
        dst.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(status.item()) == 0
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=2048, sizes=sizes_np, epoch_len=1000, tile_bytes=tile)
        assert sched.table_numpy().tobytes() == exp_t.tobytes(), f"replay {rep}"
        np.testing.assert_array_equal(dst.cpu().numpy()[:total], src_np[:total], err_msg=f"replay {rep}")
        assert not dst[total:].any()


@pytest.mark.parametrize("seed", range(12))
def test_one_scheduler_launch_for_a_message_that_moves_in_waves(fl, seed):
    """wave_chunks: the rows of wave w are what a call for that wave alone (offsets from zero, state carried from the
    wave before) writes -- the oracle is run wave by wave -- while header and state are the whole call's; the copies
    driven wave by wave over windows that hold one wave round-trip the message."""
    core, torch = fl
    rng = np.random.default_rng(6200 + seed)
    lanes = int(rng.integers(1, 17))
    rows = int(rng.integers(1, 5))
    credits = rng.integers(0, 9, size=(rows, lanes)).astype(np.uint32)
    epoch_len = int(rng.choice([0, 7, 50, 1000]))
    chunk = int(rng.choice([4096, 8192 + 128, 65536]))
    n = int(rng.integers(1, 900))
    V = int(rng.choice([1, 5, 64, 100, 1000]))
    total = n * chunk - int(rng.integers(0, chunk))
    tile = int(rng.choice([128, 4096, 32768]))
    st0 = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    if seed % 2:
        st0["epoch_bytes"] = int(rng.integers(0, 40)) * chunk
        st0["chunk_index"] = int(rng.integers(0, 3000))
        st0["lane_off"][:lanes] = rng.integers(0, 1 << 20, size=lanes)
    # expectation: the oracle wave by wave
    st = st0.copy()
    exp_rows, need = [], np.zeros(lanes, dtype=np.int64)
    for w0 in range(0, n, V):
        lo, hi = w0 * chunk, min(total, (w0 + V) * chunk)
        t_w, h_w, st = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=hi - lo, chunk_bytes=chunk, src_base=lo,
                                          epoch_len=epoch_len, tile_bytes=tile, mode=(0 if w0 == 0 else ob.SCHED_RESET_OFFSETS), state=st)
        exp_rows.append(t_w)
        if w0:
            need = np.maximum(need, h_w["lane_bytes"][:lanes].astype(np.int64))
        else:
            need = np.maximum(need, st0["lane_off"][:lanes].astype(np.int64) + h_w["lane_bytes"][:lanes].astype(np.int64))
    exp_t = np.concatenate(exp_rows)
    whole_t, whole_h, whole_s = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                                   epoch_len=epoch_len, tile_bytes=tile, state=st0.copy())
    d_state = _dev(torch, np.array([st0], dtype=ob.STATE_DTYPE).view(np.uint8))
    sched = core.schedule(n_lanes=lanes, credits=_dev(torch, credits.view(np.int32)), quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                          epoch_len=epoch_len, tile_bytes=tile, state=d_state, wave_chunks=V)
    torch.cuda.synchronize()
    got_t, got_h = sched.table_numpy(), sched.hdr_numpy()
    for f in ("src_off", "win_off", "len", "lane", "epoch"):
        np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f"table field {f}")
    np.testing.assert_array_equal(got_t["tile_base"], whole_t["tile_base"])
    for f in ("total_bytes", "total_tiles", "n_chunks", "flags", "uniform_tiles", "lane_bytes", "lane_chunks"):
        np.testing.assert_array_equal(got_h[f], whole_h[f], err_msg=f"hdr field {f}")
    got_s = core.state_numpy(d_state)
    for f in ("epoch_bytes", "chunk_index"):
        assert got_s[f] == whole_s[f], f
    np.testing.assert_array_equal(got_s["lane_off"], whole_s["lane_off"])
    # the copies, wave by wave, over windows that hold one wave
    caps = [int(x) for x in need]
    wins = [torch.zeros(max(c, 1), dtype=torch.uint8, device="cuda") for c in caps]
    w = core.make_windows([t.data_ptr() for t in wins], caps)
    src = torch.randint(0, 256, (total,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    status = core.new_status()
    row_bytes = core.DESC_DTYPE.itemsize
    for w0 in range(0, n, V):
        cnt = min(V, n - w0)
        lo, hi = w0 * chunk, min(total, (w0 + V) * chunk)
        sub = core.Schedule(sched.table[w0 * row_bytes:], sched.hdr, cnt, tile)
        hint = core.uniform_hint(hi - lo, chunk, tile)
        core.stripe(src, w, sub, status, hint=hint)
        core.reassemble(dst, w, sub, status, hint=hint)
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and torch.equal(src, dst)


@pytest.mark.parametrize("xcd_runs", [1, 0])
@pytest.mark.parametrize("seed", range(6))
def test_copies_with_tiles_taken_in_runs_per_xcd(fl, seed, xcd_runs):
    """Grids of 256 workgroups and more hand each XCD runs of 32 consecutive tiles instead of every eighth tile.  The
    map only changes which workgroup copies which tile: messages of several hundred small tiles (whole blocks of 256
    and a ragged rest, tile counts per chunk that are powers of two and ones that are not) through the fused pair, the
    table-driven pair with and without the host's header, the descriptor-driven pair and the plain copy, against the
    oracle, with the map on and off."""
    core, torch = fl
    rng = np.random.default_rng(7300 + seed)
    core.tune("xcd_runs", xcd_runs)
    try:
        lanes = int(rng.integers(1, 17))
        tile = int(rng.choice([128, 256, 1024]))
        tpc = int(rng.choice([1, 2, 4, 8, 16, 3, 6]))
        chunk = tile * tpc
        n = int(rng.integers(300, 2500)) // tpc + 1
        total = n * chunk - int(rng.integers(0, chunk))
        credits = rng.integers(0, 9, size=lanes).astype(np.uint32)
        credits[int(rng.integers(0, lanes))] = 5
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                                             tile_bytes=tile, mode=ob.SCHED_RESET_OFFSETS)
        assert int(exp_h["total_tiles"]) >= 256
        src_np = rng.integers(0, 256, size=total, dtype=np.uint8)
        src = _dev(torch, src_np)
        caps = [int(b) for b in exp_h["lane_bytes"][:lanes]]
        exp_w = ob.cpu_stripe(src_np, exp_t, caps)

        def fresh():
            wins = [torch.zeros(max(c, 1) + 64, dtype=torch.uint8, device="cuda") for c in caps]
            return wins, core.make_windows([t.data_ptr() for t in wins], caps)

        def check(wins, dst, what):
            torch.cuda.synchronize()
            assert int(status.item()) == 0, what
            for l in range(lanes):
                got = wins[l].cpu().numpy()
                np.testing.assert_array_equal(got[: caps[l]], exp_w[l][: caps[l]], err_msg=f"{what}, lane {l}")
                assert not got[caps[l]:].any(), what
            np.testing.assert_array_equal(dst.cpu().numpy(), src_np, err_msg=what)

        status = core.new_status()
        # scheduler folded into the copies
        u = core.uniform_params(total, chunk, credits, tile_bytes=tile)
        out = core.new_schedule_buffers(n, tile)
        wins, w = fresh()
        dst = torch.zeros_like(src)
        core.stripe_uniform(src, w, u, status, out=out)
        core.reassemble_uniform(dst, w, u, status)
        check(wins, dst, "fused")
        got_t, got_h = out.table_numpy(), out.hdr_numpy()
        for f in ob.DESC_DTYPE.names:
            np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f)
        for f in ("total_bytes", "total_tiles", "n_chunks", "uniform_tiles", "lane_bytes", "lane_chunks"):
            np.testing.assert_array_equal(got_h[f], exp_h[f], err_msg=f)
        # table-driven: the search kernel (no host header), the two-dimensional grid (host header), the descriptors
        sched = core.schedule(n_lanes=lanes, credits=[int(c) for c in credits], quantum=chunk, total_bytes=total, chunk_bytes=chunk,
                              tile_bytes=tile, mode=core.SCHED_RESET_OFFSETS, tiles_capacity=int(exp_h["total_tiles"]) + 3)
        torch.cuda.synchronize()
        hint = core.uniform_hint(total, chunk, tile)
        plain = core.Schedule(sched.table, sched.hdr, n, tile)
        for what, s_, h_ in (("search", plain, None), ("grid", plain, hint), ("descriptors", sched, hint), ("descriptors, device header", sched, None)):
            wins, w = fresh()
            dst = torch.zeros_like(src)
            core.stripe(src, w, s_, status, hint=h_)
            core.reassemble(dst, w, s_, status, hint=h_)
            check(wins, dst, what)
        # the calibration copy
        big = torch.randint(0, 256, (300 * core.TILE_BYTES + 77,), dtype=torch.uint8, device="cuda")
        back = torch.zeros_like(big)
        core.copy(back, big)
        torch.cuda.synchronize()
        assert torch.equal(back, big)
    finally:
        core.tune("xcd_runs", 1)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(6))
def test_runs_of_several_lanes_in_one_launch(fl, seed):
    """flh_copy_runs: what carries every lane's staged bytes from one set of windows to another in a single launch.
    Runs of any length (none, a few bytes, ragged, megabytes), misaligned against each other, in any of the 16 slots;
    every destination is compared with numpy, and the bytes around every run must stay untouched."""
    core, torch = fl
    rng = np.random.default_rng(6100 + seed)
    n = int(rng.integers(1, 17))
    lens = [int(rng.choice([0, 0, int(rng.integers(1, 100)), int(rng.integers(1, 200000)), int(rng.integers(1, 5)) * (1 << 20) + int(rng.integers(0, 3)) * 7]))
            for _ in range(n)]
    if seed == 0:
        lens = [0] * n            # nothing at all: no launch, no error
    pad = 64
    srcs_np = [rng.integers(1, 256, size=ln + 2 * pad, dtype=np.uint8) for ln in lens]
    so = [int(rng.integers(0, pad)) for _ in lens]
    do = [int(rng.integers(0, pad)) for _ in lens]
    srcs = [torch.from_numpy(a).cuda() for a in srcs_np]
    dsts = [torch.zeros(ln + 2 * pad, dtype=torch.uint8, device="cuda") for ln in lens]
    core.copy_runs([d[o:] if ln else None for d, o, ln in zip(dsts, do, lens)], [s[o:] if ln else None for s, o, ln in zip(srcs, so, lens)], lens)
    torch.cuda.synchronize()
    for k, ln in enumerate(lens):
        exp = np.zeros(ln + 2 * pad, dtype=np.uint8)
        exp[do[k]:do[k] + ln] = srcs_np[k][so[k]:so[k] + ln]
        np.testing.assert_array_equal(dsts[k].cpu().numpy(), exp, err_msg=f"run {k} of {lens}")
    with pytest.raises(Exception):
        core.copy_runs([dsts[0]] * 17, [srcs[0]] * 17, [1] * 17)
