"""The plugin ABI with device memory on a real MI355X: isend/irecv/test drive the scheduler,
striping and reassembly kernels through HIP-VMM staging windows; results are compared with the CPU
oracle (chunk -> lane tables bit-exact, reassembled buffers bit-exact)."""
import numpy as np
import pytest

from fuselink_amd import plugin as P
from tests import oracle_binding as ob

pytestmark = pytest.mark.gpu

ENV_KEYS = ["NCCL_FUSELINK_LANES", "NCCL_FUSELINK_CHUNKSIZE", "NCCL_FUSELINK_POLICY", "NCCL_FUSELINK_WINDOW_UNITS",
            "NCCL_FUSELINK_POOL_UNITS", "NCCL_FUSELINK_REFRESH_BATCH", "NCCL_IB_QPS_PER_CONNECTION", "NCCL_FUSELINK_CREDITS",
            "NCCL_FUSELINK_BATCH", "NCCL_FUSELINK_COMPLETION", "NCCL_FUSELINK_ENGINE", "NCCL_FUSELINK_ENGINE_SETS", "NCCL_FUSELINK_ENGINE_UNITS",
            "NCCL_FUSELINK_ONE_PASS"]


@pytest.fixture()
def net():
    import torch
    p = P.NetPlugin(8)
    p.reconfigure(**{k: None for k in ENV_KEYS})
    p.lib.fl_monitor_reset()
    p.set_credits([])
    yield p
    torch.cuda.synchronize()
    p.reconfigure(**{k: None for k in ENV_KEYS})


def _send_recv(net, s, r, src, dst, size, tag, smh, rmh, src_off=0, dst_off=0):
    rc, rreq = net.irecv(r, [dst.data_ptr() + dst_off], [size], [tag], [rmh])
    assert rc == 0 and rreq
    rc, sreq = net.isend(s, src.data_ptr() + src_off, size, tag, smh)
    assert rc == 0 and sreq
    net.wait(sreq)
    assert net.wait(rreq) == size


def test_cfg1_shape_on_gpu(net):
    # 4 MiB uint8, 512 KiB chunks, 2 lanes, equal credits: lanes 0,1,0,1,... and one 2 MiB unit per lane
    import torch
    net.reconfigure(NCCL_FUSELINK_LANES=2, NCCL_FUSELINK_CHUNKSIZE=512 << 10, NCCL_FUSELINK_WINDOW_UNITS=1)
    net.set_credits([1, 1])
    rng = np.random.default_rng(1)
    src_np = rng.integers(0, 256, size=4 << 20, dtype=np.uint8)
    src = torch.from_numpy(src_np).cuda()
    dst = torch.zeros_like(src)
    lcomm, s, r = net.connect_pair(0)
    rc, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
    assert rc == 0
    rc, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
    assert rc == 0
    _send_recv(net, s, r, src, dst, 4 << 20, 5, smh, rmh)
    np.testing.assert_array_equal(dst.cpu().numpy(), src_np)
    rows, hdr = net.last_table(s)
    # a 2 MiB window holds 4 chunks and each lane gets exactly 4 of the 8: the whole request is one wave
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=2, credits=[1, 1], quantum=512 << 10, total_bytes=4 << 20,
                                         chunk_bytes=512 << 10, mode=ob.SCHED_RESET_OFFSETS)
    _same_table(rows, exp_t)
    assert [int(b) for b in exp_h["lane_bytes"][:2]] == [2 << 20, 2 << 20]
    # a second request starts one quantum further on in the slot cycle only if the first left it there: 8 chunks
    # over 2 lanes end on a whole round, so 5 more chunks (2.5 MiB) go 3 + 2 and still fit one wave
    src2, dst2 = src[: 5 * (512 << 10)], dst[: 5 * (512 << 10)]
    dst.zero_()
    _send_recv(net, s, r, src2, dst2, 5 * (512 << 10), 6, smh, rmh)
    np.testing.assert_array_equal(dst2.cpu().numpy(), src_np[: 5 * (512 << 10)])
    rows, hdr = net.last_table(s)
    exp_t, _, _ = ob.credit_schedule(n_lanes=2, credits=[1, 1], quantum=512 << 10, total_bytes=5 * (512 << 10),
                                     chunk_bytes=512 << 10, mode=ob.SCHED_RESET_OFFSETS, state=_state(4 << 20, 8))
    _same_table(rows, exp_t)
    # 12 chunks do not fit 2 x 4: from quantum 13 on the lanes alternate, so 8 chunks fill both windows and 4 follow
    big_np = rng.integers(0, 256, size=6 << 20, dtype=np.uint8)
    big, back = torch.from_numpy(big_np).cuda(), torch.zeros(6 << 20, dtype=torch.uint8, device="cuda")
    rc, bmh = net.regMr(s, big.data_ptr(), big.numel(), P.NCCL_PTR_CUDA)
    assert rc == 0
    rc, kmh = net.regMr(r, back.data_ptr(), back.numel(), P.NCCL_PTR_CUDA)
    assert rc == 0
    _send_recv(net, s, r, big, back, 6 << 20, 7, bmh, kmh)
    np.testing.assert_array_equal(back.cpu().numpy(), big_np)
    rows, hdr = net.last_table(s)
    exp_t, _, _ = ob.credit_schedule(n_lanes=2, credits=[1, 1], quantum=512 << 10, total_bytes=4 * (512 << 10), chunk_bytes=512 << 10,
                                     src_base=8 * (512 << 10), mode=ob.SCHED_RESET_OFFSETS, state=_state(21 * (512 << 10), 21))
    _same_table(rows, exp_t)
    assert net.deregMr(s, bmh) == 0 and net.deregMr(r, kmh) == 0
    assert net.deregMr(s, smh) == 0 and net.deregMr(r, rmh) == 0
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def _state(epoch_bytes, chunk_index):
    st = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    st["epoch_bytes"] = epoch_bytes
    st["chunk_index"] = chunk_index
    return st


def _same_table(got, exp):
    assert got.size == exp.size
    for f in ob.DESC_DTYPE.names:
        np.testing.assert_array_equal(got[f], exp[f], err_msg=f)


def test_cfg2_shape_through_plugin(net):
    # 64 MiB fp16 N(0,1), 256 KiB chunks, 8 lanes, credits uniform in [1,8]; one wave holds the message
    import torch
    rng = np.random.default_rng(2)
    credits = [int(c) for c in rng.integers(1, 9, size=8)]
    net.reconfigure(NCCL_FUSELINK_LANES=8, NCCL_FUSELINK_CHUNKSIZE=256 << 10, NCCL_FUSELINK_WINDOW_UNITS=28)
    net.set_credits(credits)
    src_np = rng.standard_normal(32 << 20, dtype=np.float32).astype(np.float16).view(np.uint8)
    src = torch.from_numpy(src_np).cuda()
    dst = torch.zeros_like(src)
    lcomm, s, r = net.connect_pair(0)
    _, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
    _, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
    _send_recv(net, s, r, src, dst, 64 << 20, 1, smh, rmh)
    np.testing.assert_array_equal(dst.cpu().numpy(), src_np)
    rows, hdr = net.last_table(s)
    W, cmax = sum(credits), max(credits)
    per_wave = ((28 * 2 * 4) // cmax - 1) * W   # chunks per wave the plugin allows itself
    n_last = 256 % per_wave or per_wave
    first = 256 - n_last
    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=8, credits=credits, quantum=256 << 10, total_bytes=n_last * (256 << 10),
                                         chunk_bytes=256 << 10, src_base=first * (256 << 10),
                                         mode=ob.SCHED_RESET_OFFSETS, state=_state(first * (256 << 10), first))
    _same_table(rows, exp_t)
    np.testing.assert_array_equal(hdr["lane_bytes"], exp_h["lane_bytes"])
    net.deregMr(s, smh), net.deregMr(r, rmh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_regMrDmaBuf_takes_a_real_dmabuf_and_checks_its_size(net):
    """regMrDmaBuf with a descriptor (src/plugin.cc:1168, 1278-1280): a DMA-BUF of device memory that holds the registered
    range is accepted and the registration works like any other; one that is too short for the range, or for the offset
    that came with it, is refused.  The descriptor here is the export of a 2 MiB staging unit (flh_window_export_dmabuf)."""
    import os

    import torch
    from fuselink_amd import core
    net.reconfigure(NCCL_FUSELINK_LANES=4, NCCL_FUSELINK_CHUNKSIZE=128 << 10)
    net.set_credits([1, 2, 1, 1])
    pool = core.Pool(0, 4)
    w = core.Window(pool, 2 << 20)
    w.bind(2 << 20)
    fd = w.export_dmabuf(0, 2 << 20)
    src = torch.randint(0, 255, (1 << 20,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    lcomm, s, r = net.connect_pair(0)
    try:
        rc, smh = net.regMrDmaBuf(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA, 0, fd)
        assert rc == 0 and smh
        rc, bad = net.regMrDmaBuf(s, src.data_ptr(), 4 << 20, P.NCCL_PTR_CUDA, 0, fd)          # 4 MiB do not fit a 2 MiB descriptor
        assert rc == P.ncclInvalidArgument and bad is None
        rc, bad = net.regMrDmaBuf(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA, (2 << 20) - 4096, fd)   # nor 1 MiB behind that offset
        assert rc == P.ncclInvalidArgument and bad is None
        rc, rmh = net.regMrDmaBuf(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA, 0, -1)
        assert rc == 0 and rmh
        os.close(fd)                                     # the registration keeps a duplicate of its own
        fd = -1
        _send_recv(net, s, r, src, dst, 1 << 20, 3, smh, rmh)
        assert torch.equal(src, dst)
        rc, props = net.getProperties(0)
        assert props.ptrSupport & P.NCCL_PTR_DMABUF
        assert net.deregMr(s, smh) == 0 and net.deregMr(r, rmh) == 0
    finally:
        if fd >= 0:
            os.close(fd)
        net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)
        w.destroy()
        pool.destroy()


def test_static_policy_puts_a_channel_on_one_lane(net):
    # the reference's live policy: lane = channelId % nNics (src/fuselink.h:235), receiver decides, sender obeys
    import torch
    net.reconfigure(NCCL_FUSELINK_LANES=4, NCCL_FUSELINK_POLICY=0, NCCL_FUSELINK_CHUNKSIZE=128 << 10)
    src = torch.randint(0, 255, (2 << 20,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    for _ in range(3):
        rc, handle, lcomm = net.listen(0)
        channel = int.from_bytes(handle.raw[16:20], "little", signed=True)
        net.closeListen(lcomm)
        lcomm, s, r = net.connect_pair(0)
        channel += 1
        _, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
        _, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
        dst.zero_()
        _send_recv(net, s, r, src, dst, 2 << 20, 0, smh, rmh)
        assert torch.equal(src, dst)
        rows, hdr = net.last_table(s)
        assert set(rows["lane"].tolist()) == {channel % 4}
        net.deregMr(s, smh), net.deregMr(r, rmh)
        net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_busy_lane_gets_no_chunks_after_refresh(net):
    """Monitor-driven credits: a lane whose NIC was active within the 160 us timeout is BUSY and is
    routed around at the next refresh (src/monitor.h:236-250, src/monitor.cpp:159-193)."""
    import torch
    net.reconfigure(NCCL_FUSELINK_LANES=4, NCCL_FUSELINK_CHUNKSIZE=64 << 10, NCCL_FUSELINK_REFRESH_BATCH=1)
    L = net.lib
    L.fl_monitor_set_clock(1, 1_000_000)
    L.fl_monitor_mark_active(2, 1, 1_000_000 - 10)     # lane 2 busy 10 us ago
    src = torch.randint(0, 255, (4 << 20,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    lcomm, s, r = net.connect_pair(0)
    _, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
    _, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
    _send_recv(net, s, r, src, dst, 4 << 20, 0, smh, rmh)
    assert torch.equal(src, dst)
    rows, hdr = net.last_table(s)
    assert hdr["lane_chunks"][2] == 0 and all(hdr["lane_chunks"][l] > 0 for l in (0, 1, 3))
    # 160 us later the lane has aged to IDLE and takes traffic again at the next refresh
    L.fl_monitor_set_clock(1, 1_000_000 + 200)
    dst.zero_()
    _send_recv(net, s, r, src, dst, 4 << 20, 1, smh, rmh)
    assert torch.equal(src, dst)
    rows, hdr = net.last_table(s)
    assert hdr["lane_chunks"][2] > 0
    L.fl_monitor_set_clock(0, 0)
    net.deregMr(s, smh), net.deregMr(r, rmh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_scheduler_reads_live_credits_from_pinned_host_memory(net):
    """The credit row the scheduler kernels read may live in pinned host memory that the monitor side rewrites
    in place: no copy, no semaphore on the request path.  fl_monitor_credits writes the row straight into the
    pinned table; the next launch sees it."""
    import ctypes as C

    import torch
    from fuselink_amd import core
    L = net.lib
    lanes, chunk, total = 8, 64 << 10, 37 * (64 << 10) - 100
    L.fl_monitor_reset()
    L.fl_monitor_set_clock(1, 5_000_000)
    row = torch.zeros(lanes, dtype=torch.int32).pin_memory()       # device-visible host memory
    row_ptr = C.cast(row.data_ptr(), C.POINTER(C.c_uint32))
    try:
        for busy in ([], [1, 6], [0, 1, 2, 3, 4, 5, 6, 7]):
            L.fl_monitor_reset()
            for l in busy:
                L.fl_monitor_mark_active(l, 1, 5_000_000 - 20)
            assert L.fl_monitor_credits(lanes, 3, 4, row_ptr) == 0    # own lane 3 never drops to zero
            credits = row.numpy().astype(np.uint32).copy()
            assert list(credits) == [0 if l in busy and l != 3 else (1 if l == 3 and 3 in busy else 4) for l in range(lanes)]
            exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=total, chunk_bytes=chunk)
            for fast in (1, 0):                                        # closed-form and scan kernels
                core.tune("sched_uniform_fast", fast)
                p = core.SchedParams()
                out = core.new_schedule_buffers(len(exp_t))
                p.total_bytes, p.chunk_bytes, p.n_chunks, p.n_lanes = total, chunk, len(exp_t), lanes
                p.d_credits, p.n_rows, p.quantum, p.tile_bytes = row.data_ptr(), 1, chunk, 32768
                p.d_table, p.d_hdr = out.table.data_ptr(), out.hdr.data_ptr()
                core.check(core._lib.load().flh_schedule(C.byref(p), None))
                torch.cuda.synchronize()
                _same_table(out.table_numpy(), exp_t)
                np.testing.assert_array_equal(out.hdr_numpy()["lane_chunks"], exp_h["lane_chunks"])
    finally:
        core.tune("sched_uniform_fast", 1)
        L.fl_monitor_set_clock(0, 0)
        L.fl_monitor_reset()


def test_stress_shape_many_requests_in_flight(net):
    """Shape of the stress configuration at a quarter of its size per step: uint32 payload, 64 KiB
    chunks, 16 lanes, credits redrawn at every refresh, 4 requests in flight, windows reused by every
    wave (16 lanes x 4 units = 64 of the pool's 256 units for 1 GiB of traffic)."""
    import torch
    net.reconfigure(NCCL_FUSELINK_LANES=16, NCCL_FUSELINK_CHUNKSIZE=64 << 10, NCCL_FUSELINK_REFRESH_BATCH=4,
                    NCCL_FUSELINK_WINDOW_UNITS=4)
    rng = np.random.default_rng(5)
    total = 1 << 30
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    src = torch.randint(0, 2**31 - 1, (total // 4,), dtype=torch.int32, device="cuda", generator=gen).view(torch.uint8)
    dst = torch.zeros_like(src)
    lcomm, s, r = net.connect_pair(0)
    _, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
    _, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
    piece = 64 << 20
    n_req = total // piece
    posted = sent = 0
    inflight = []
    net.set_credits([int(c) for c in rng.integers(1, 9, size=16)])
    while sent < n_req or inflight:
        progressed = False
        if posted < n_req and posted - sent < 4:
            before = net.comm_stats(r)["refreshes"]
            rc, rreq = net.irecv(r, [dst.data_ptr() + posted * piece], [piece], [posted], [rmh])
            assert rc == 0
            if rreq:
                if net.comm_stats(r)["refreshes"] != before:   # the lane decision was refreshed: redraw for the next one
                    net.set_credits([int(c) for c in rng.integers(1, 9, size=16)])
                inflight.append(("r", rreq))
                posted += 1
                progressed = True
        if sent < posted:
            rc, sreq = net.isend(s, src.data_ptr() + sent * piece, piece, sent, smh)
            assert rc == 0
            if sreq:
                inflight.append(("s", sreq))
                sent += 1
                progressed = True
        still = []
        for kind, q in inflight:
            rc, done, size = net.test(q)
            assert rc == 0
            if done:
                progressed = True
                if kind == "r":
                    assert size == piece
            else:
                still.append((kind, q))
        inflight = still
    torch.cuda.synchronize()
    assert torch.equal(src, dst)
    st = net.comm_stats(r)
    # a refresh needs an irecv to arrive exactly on a batch boundary with nothing outstanding
    # (src/plugin.cc:1700-1712); with requests posted ahead some boundaries pass unseen
    assert st["n_finished"] == n_req and 1 <= st["refreshes"] <= n_req // 4 + 1
    net.deregMr(s, smh), net.deregMr(r, rmh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_qp_split_and_ragged_sizes(net):
    # request -> 3 QP pieces of 128-byte-aligned stride (src/plugin.cc:1467-1495), each chunked on its own
    import torch
    net.reconfigure(NCCL_FUSELINK_LANES=3, NCCL_FUSELINK_CHUNKSIZE=4096, NCCL_IB_QPS_PER_CONNECTION=3)
    net.set_credits([2, 1, 1])
    for size in (1, 100, 1000, 4097, 1000003):
        src = torch.randint(0, 255, (size + 64,), dtype=torch.uint8, device="cuda")
        dst = torch.zeros_like(src)
        lcomm, s, r = net.connect_pair(0)
        _, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
        _, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
        _send_recv(net, s, r, src, dst, size, 3, smh, rmh)
        assert torch.equal(src[:size], dst[:size]) and not dst[size:].any()
        net.deregMr(s, smh), net.deregMr(r, rmh)
        net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_mixed_host_and_device_buffers(net):
    import torch
    src = torch.randint(0, 255, (1 << 20,), dtype=torch.uint8, device="cuda")
    host = np.zeros(1 << 20, dtype=np.uint8)
    lcomm, s, r = net.connect_pair(0)
    _, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
    _, rmh = net.regMr(r, host.ctypes.data, host.size, P.NCCL_PTR_HOST)
    rc, rreq = net.irecv(r, [host.ctypes.data], [1 << 20], [0], [rmh])
    rc, sreq = net.isend(s, src.data_ptr(), 1 << 20, 0, smh)
    assert rc == 0 and sreq
    net.wait(sreq), net.wait(rreq)
    np.testing.assert_array_equal(host, src.cpu().numpy())
    net.deregMr(s, smh), net.deregMr(r, rmh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


@pytest.mark.parametrize("completion,engine,one_pass", [(0, 0, 1), (1, 0, 1), (2, 0, 1), (2, 1, 1), (0, 0, 0), (1, 0, 0), (2, 0, 0)])
@pytest.mark.parametrize("batch", [1, 8])
def test_completion_reaches_test_in_every_mode(net, completion, engine, one_pass, batch):
    """How `test` learns that a launch is done -- an event behind every launch, an event on the launch's last kernel,
    the words that kernels store launch numbers to (a small launch's reassembly kernel when its last workgroup has
    finished, every striping kernel as it starts, an event only behind a large launch that nothing follows), or the
    lane engine's completion word for the small requests it carries -- must not change what a consumer sees, whether a
    launch stages and delivers in one kernel (one_pass) or a striping and a reassembly kernel do: every receive is compared on torch's own stream, which does not wait for the
    connection's, the moment `test` reports it done, with requests in flight behind it, empty requests and host
    buffers mixed in, and a lone request at the end that no other launch follows."""
    import torch
    net.reconfigure(NCCL_FUSELINK_LANES=4, NCCL_FUSELINK_CHUNKSIZE=64 << 10, NCCL_FUSELINK_WINDOW_UNITS=1,
                    NCCL_FUSELINK_BATCH=batch, NCCL_FUSELINK_COMPLETION=completion, NCCL_FUSELINK_ENGINE=engine, NCCL_FUSELINK_ONE_PASS=one_pass)
    net.set_credits([3, 1, 2, 2])
    rng = np.random.default_rng(900 + completion * 10 + batch)
    n_req = 120
    sizes = [int(rng.choice([0, 1, 4096, 64 << 10, 200000, 1 << 20, (3 << 20) + 17])) for _ in range(n_req)]
    kinds = ["host" if rng.random() < 0.1 else "dev" for _ in range(n_req)]
    offs = np.concatenate([[0], np.cumsum([(x + 255) // 256 * 256 for x in sizes])])
    total = int(offs[-1]) + 256
    src = torch.randint(0, 256, (total,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    host_dst = np.zeros(total, dtype=np.uint8)
    lcomm, s, r = net.connect_pair(0)
    _, smh = net.regMr(s, src.data_ptr(), total, P.NCCL_PTR_CUDA)
    _, rmh = net.regMr(r, dst.data_ptr(), total, P.NCCL_PTR_CUDA)
    _, hmh = net.regMr(r, host_dst.ctypes.data, total, P.NCCL_PTR_HOST)
    src_np = src.cpu().numpy()
    posted = sent = checked = 0
    rq, sq = [], []
    depth = 6
    while checked < n_req:
        if posted < n_req and len(rq) < depth:
            k, o = posted, int(offs[posted])
            if kinds[k] == "host":
                rc, rreq = net.irecv(r, [host_dst.ctypes.data + o], [sizes[k]], [k], [hmh])
            else:
                rc, rreq = net.irecv(r, [dst.data_ptr() + o], [sizes[k]], [k], [rmh])
            assert rc == 0
            if rreq:
                rq.append((k, rreq))
                posted += 1
        if sent < posted and len(sq) < depth:
            rc, sreq = net.isend(s, src.data_ptr() + int(offs[sent]), sizes[sent], sent, smh)
            assert rc == 0
            if sreq:
                sq.append(sreq)
                sent += 1
        if sq:
            rc, done, _ = net.test(sq[0])
            assert rc == 0
            if done:
                sq.pop(0)
        if rq:
            k, rreq = rq[0]
            rc, done, size = net.test(rreq)
            assert rc == 0
            if done:
                assert size == sizes[k]
                o = int(offs[k])
                if kinds[k] == "host":
                    np.testing.assert_array_equal(host_dst[o: o + sizes[k]], src_np[o: o + sizes[k]], err_msg=f"request {k}")
                else:   # a kernel on another stream, started at once
                    assert torch.equal(dst[o: o + sizes[k]], src[o: o + sizes[k]]), f"request {k} of {sizes[k]} bytes"
                rq.pop(0)
                checked += 1
    # one request alone on an idle connection: nothing follows its launch
    for size in (1 << 20, 5):
        dst.zero_()
        _send_recv(net, s, r, src, dst, size, 1000 + size, smh, rmh)
        assert torch.equal(dst[:size], src[:size]) and not dst[size:].any()
    net.deregMr(s, smh), net.deregMr(r, rmh), net.deregMr(r, hmh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_region_is_shared_and_refcounted(net):
    # k registrations of the same allocation share one region; it dies with the k-th deregistration
    # (src/plugin.cc:1212-1227, 1337-1408)
    import torch
    buf = torch.zeros(8 << 20, dtype=torch.uint8, device="cuda")
    lcomm, s, r = net.connect_pair(0)
    hs = []
    for off in (0, 4096, 1 << 20):
        rc, mh = net.regMr(r, buf.data_ptr() + off, 4096, P.NCCL_PTR_CUDA)
        assert rc == 0 and mh
        hs.append(mh)
    assert len(set(hs)) == 3
    for mh in hs:
        assert net.deregMr(r, mh) == 0
    rc, mh = net.regMr(r, buf.data_ptr(), 4096, P.NCCL_PTR_CUDA)
    assert rc == 0
    net.deregMr(r, mh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_largest_request_an_int_can_name(net):
    # isend/irecv sizes are `int` (src/extern/nccl_net.h:74): 2 GiB - 1 bytes in one request, waves reuse the windows
    import torch
    size = (1 << 31) - 1
    net.reconfigure(NCCL_FUSELINK_LANES=16, NCCL_FUSELINK_CHUNKSIZE=512 << 10, NCCL_FUSELINK_WINDOW_UNITS=4)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(9)
    src = torch.randint(0, 2**31 - 1, ((1 << 31) // 4,), dtype=torch.int32, device="cuda", generator=gen).view(torch.uint8)
    dst = torch.zeros_like(src)
    lcomm, s, r = net.connect_pair(0)
    _, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
    _, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
    _send_recv(net, s, r, src, dst, size, 11, smh, rmh)
    assert torch.equal(src[:size], dst[:size]) and int(dst[size]) == 0
    net.deregMr(s, smh), net.deregMr(r, rmh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_epoch_prefix_carries_across_requests_until_refresh(net):
    """The byte prefix that picks the slot runs on from request to request and restarts when the receiver
    refreshes its lane decision (every REFRESH_BATCH completions): tables against the oracle's carried state."""
    import torch
    chunk = 64 << 10
    net.reconfigure(NCCL_FUSELINK_LANES=4, NCCL_FUSELINK_CHUNKSIZE=chunk, NCCL_FUSELINK_REFRESH_BATCH=3)
    credits = [3, 1, 2, 2]
    net.set_credits(credits)
    src = torch.randint(0, 255, (4 << 20,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    lcomm, s, r = net.connect_pair(0)
    _, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
    _, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
    sizes = [5 * chunk, 3 * chunk + 100, 7 * chunk, 2 * chunk, 9 * chunk - 1, chunk, 4 * chunk]
    prefix = 0
    for k, size in enumerate(sizes):
        if k % 3 == 0:
            prefix = 0                      # refresh: a new credit epoch
        dst.zero_()
        _send_recv(net, s, r, src, dst, size, k, smh, rmh)
        assert torch.equal(src[:size], dst[:size])
        rows, hdr = net.last_table(s)
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=4, credits=credits, quantum=chunk, total_bytes=size, chunk_bytes=chunk,
                                             mode=ob.SCHED_RESET_OFFSETS, state=_state(prefix, 0))
        _same_table(rows, exp_t)
        np.testing.assert_array_equal(hdr["lane_bytes"], exp_h["lane_bytes"])
        prefix += size
    net.deregMr(s, smh), net.deregMr(r, rmh)
    net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


def test_sends_that_wait_together_travel_as_one_message(net):
    """Seven 512 KiB requests posted before anything is tested: one launch pair carries them all, scheduled as
    the 3.5 MiB message they form (table against the oracle), every receive buffer gets its own data; with
    NCCL_FUSELINK_BATCH=1 the same traffic takes one launch pair per request and gives the same bytes.
    (A first request goes alone: on a refresh boundary the reference's gate admits one receive at a time.)"""
    import torch
    rng = np.random.default_rng(77)
    chunk, piece, n_req = 64 << 10, 512 << 10, 7
    credits = [3, 1, 0, 2, 5, 1, 1, 4]
    src_np = rng.integers(0, 256, size=(n_req + 1) * piece, dtype=np.uint8)
    src = torch.from_numpy(src_np).cuda()
    for batch, exp_launches, exp_batched in ((8, 1, 7), (1, 7, 0), (3, 3, 6)):
        net.reconfigure(NCCL_FUSELINK_LANES=8, NCCL_FUSELINK_CHUNKSIZE=chunk, NCCL_FUSELINK_BATCH=batch)
        net.set_credits(credits)
        dst = torch.zeros_like(src)
        lcomm, s, r = net.connect_pair(0)
        _, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
        _, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
        _send_recv(net, s, r, src, dst, piece, 99, smh, rmh, src_off=n_req * piece, dst_off=n_req * piece)
        assert net.launch_stats(s) == {"launches": 1, "batched_requests": 0}
        rreqs, sreqs = [], []
        # receive buffers in reverse order, so that a batch has to route every request to its own buffer
        for k in range(n_req):
            rc, q = net.irecv(r, [dst.data_ptr() + (n_req - 1 - k) * piece], [piece], [k], [rmh])
            assert rc == 0 and q
            rreqs.append(q)
        for k in range(n_req):
            rc, q = net.isend(s, src.data_ptr() + k * piece, piece, k, smh)
            assert rc == 0 and q
            sreqs.append(q)
        for q in sreqs:
            net.wait(q)
        for q in rreqs:
            assert net.wait(q) == piece
        st = net.launch_stats(s)
        assert st == {"launches": 1 + exp_launches, "batched_requests": exp_batched}, st
        got = dst.cpu().numpy().reshape(n_req + 1, piece)
        for k in range(n_req):
            np.testing.assert_array_equal(got[n_req - 1 - k], src_np[k * piece:(k + 1) * piece])
        np.testing.assert_array_equal(got[n_req], src_np[n_req * piece:])
        if batch == 8:
            rows, hdr = net.last_table(s)
            exp_t, exp_h, _ = ob.credit_schedule(n_lanes=8, credits=credits, quantum=chunk, total_bytes=n_req * piece,
                                                 chunk_bytes=chunk, mode=ob.SCHED_RESET_OFFSETS, state=_state(piece, 8))
            _same_table(rows, exp_t)
            np.testing.assert_array_equal(hdr["lane_bytes"], exp_h["lane_bytes"])
        net.deregMr(s, smh), net.deregMr(r, rmh)
        net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)
    net.reconfigure(NCCL_FUSELINK_BATCH=None)


def test_cfg5_stress_as_the_plugin_is_driven(net):
    """The stress configuration in the shape a communication library drives it: 1 GiB of uint32 as 16 384 requests of one
    64 KiB chunk each, 4 outstanding, 16 lanes, the lane decision refreshed every 1000 requests with credits redrawn at
    every refresh, 4 staging units per lane reused by every launch.  At two refresh boundaries the rows of the
    connection's latest launch are compared with the oracle's table for the same carried state: the last launch of an
    epoch (prefix = everything the epoch has scheduled) and the first of the next (prefix 0, new credit row)."""
    import torch
    chunk, lanes, refresh, n_req, inflight_max = 64 << 10, 16, 1000, 16384, 4
    net.reconfigure(NCCL_FUSELINK_LANES=lanes, NCCL_FUSELINK_CHUNKSIZE=chunk, NCCL_FUSELINK_REFRESH_BATCH=refresh,
                    NCCL_FUSELINK_WINDOW_UNITS=4)
    rng = np.random.default_rng(5)
    rows = rng.integers(1, 9, size=(n_req // refresh + 2, lanes))
    total = n_req * chunk
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    src = torch.randint(0, 2**31 - 1, (total // 4,), dtype=torch.int32, device="cuda", generator=gen).view(torch.uint8)
    dst = torch.zeros_like(src)
    c = _open(net, 0, src, dst)
    s, r = c["s"], c["r"]
    net.set_credits([int(x) for x in rows[0]])
    posted = sent = done_r = done_s = 0
    epoch = -1                       # credit epochs seen so far - 1 = index of the row in force
    sent_in_epoch = 0
    rq, sq = [], []
    checked = []
    spins = 0
    while done_r < n_req or done_s < n_req:
        spins += 1
        assert spins < 3_000_000, "no progress"
        # The reference's gate refreshes only when a receive is posted while the completion count stands on a multiple of
        # the cadence and nothing is outstanding (src/plugin.cc:1700-1712), so the driver drains before every 1000th post.
        if posted < n_req and posted - done_r < inflight_max and (posted % refresh != 0 or done_r == posted):
            rc, q = net.irecv(r, [dst.data_ptr() + posted * chunk], [chunk], [posted & 0xffff], [c["rmh"]])
            assert rc == 0
            if q:
                if posted % refresh == 0:      # this receive refreshed the lane decision: the next refresh draws the next row
                    assert net.comm_stats(r)["refreshes"] == posted // refresh + 1
                    net.set_credits([int(x) for x in rows[posted // refresh + 1]])
                rq.append(q)
                posted += 1
        if sent < posted:
            rc, q = net.isend(s, src.data_ptr() + sent * chunk, chunk, sent & 0xffff, c["smh"])
            assert rc == 0
            if q:
                if sent % refresh == 0:
                    epoch, sent_in_epoch = epoch + 1, 0
                sq.append(q)
                sent += 1
                sent_in_epoch += 1
                # the last send of epoch 2 and the first of epoch 3; the last of epoch 9 and the first of epoch 10
                if sent in (3 * refresh, 3 * refresh + 1, 10 * refresh, 10 * refresh + 1):
                    got, hdr = net.last_table(s)
                    n = got.size
                    assert 1 <= n <= inflight_max
                    exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=rows[epoch], quantum=chunk, total_bytes=n * chunk, chunk_bytes=chunk,
                                                         mode=ob.SCHED_RESET_OFFSETS, state=_state((sent_in_epoch - n) * chunk, 0))
                    _same_table(got, exp_t)
                    np.testing.assert_array_equal(hdr["lane_bytes"], exp_h["lane_bytes"])
                    checked.append((sent, epoch, n))
        if rq:
            rc, d, sz = net.test(rq[0])
            assert rc == 0
            if d:
                assert sz == chunk
                rq.pop(0)
                done_r += 1
        if sq:
            rc, d, _ = net.test(sq[0])
            assert rc == 0
            if d:
                sq.pop(0)
                done_s += 1
    assert [x[0] for x in checked] == [3 * refresh, 3 * refresh + 1, 10 * refresh, 10 * refresh + 1]
    assert checked[1][2] == 1 and checked[3][2] == 1      # a refresh admits one receive at a time: the epoch's first launch carries one request
    assert net.comm_stats(r)["refreshes"] == (n_req + refresh - 1) // refresh
    torch.cuda.synchronize()
    assert torch.equal(src, dst)
    _close(net, c)


def _open(net, dev, src, dst):
    lcomm, s, r = net.connect_pair(dev)
    rc, smh = net.regMr(s, src.data_ptr(), src.numel(), P.NCCL_PTR_CUDA)
    assert rc == 0
    rc, rmh = net.regMr(r, dst.data_ptr(), dst.numel(), P.NCCL_PTR_CUDA)
    assert rc == 0
    return dict(l=lcomm, s=s, r=r, smh=smh, rmh=rmh, src=src, dst=dst)


def _close(net, c):
    assert net.deregMr(c["s"], c["smh"]) == 0 and net.deregMr(c["r"], c["rmh"]) == 0
    net.closeSend(c["s"]), net.closeRecv(c["r"]), net.closeListen(c["l"])


def test_requests_of_four_connections_share_one_launch_pair(net):
    """NCCL's shape: four channels to a peer, eight requests in flight on each (experiments/bw_test/run_bw_test.sbatch:39-44;
    src/fuselink.h:14), all sharing the lanes (src/fuselink.h:271-272).  The 32 matched sends go out as ONE launch pair of
    four segments; every segment's rows are the oracle's table for that connection's message -- its own credit row, its own
    place in its credit epoch -- shifted to where the earlier segments left each lane's window, and every byte arrives."""
    import torch
    chunk, piece, n_conn, per_conn = 64 << 10, 128 << 10, 4, 8
    net.reconfigure(NCCL_FUSELINK_LANES=8, NCCL_FUSELINK_CHUNKSIZE=chunk, NCCL_FUSELINK_BATCH=32)
    rng = np.random.default_rng(4242)
    rows = [[3, 1, 0, 2, 5, 1, 1, 4], [1, 1, 1, 1, 1, 1, 1, 1], [0, 0, 7, 0, 0, 0, 0, 0], [2, 0, 2, 0, 2, 0, 2, 9]]
    conns = []
    for k in range(n_conn):
        src_np = rng.integers(0, 256, size=(per_conn + 1) * piece, dtype=np.uint8)
        c = _open(net, k % 8, torch.from_numpy(src_np).cuda(), torch.zeros((per_conn + 1) * piece, dtype=torch.uint8, device="cuda"))
        c["src_np"] = src_np
        net.set_credits(rows[k])           # the row this connection's receiver advertises at its first refresh
        _send_recv(net, c["s"], c["r"], c["src"], c["dst"], piece, 99, c["smh"], c["rmh"], src_off=per_conn * piece, dst_off=per_conn * piece)
        conns.append(c)
    rreqs, sreqs = [], []
    for c in conns:
        for q in range(per_conn):
            rc, req = net.irecv(c["r"], [c["dst"].data_ptr() + q * piece], [piece], [q], [c["rmh"]])
            assert rc == 0 and req
            rreqs.append(req)
    for c in conns:                        # the 32nd send fills the launch: it goes out inside that isend
        for q in range(per_conn):
            rc, req = net.isend(c["s"], c["src"].data_ptr() + q * piece, piece, q, c["smh"])
            assert rc == 0 and req
            sreqs.append(req)
    segs, got, hdr = net.last_launch(conns[0]["s"])
    assert len(segs) == n_conn and [s["n_req"] for s in segs] == [per_conn] * n_conn
    tiles_per_chunk = chunk // 32768
    lane_end = np.zeros(16, dtype=np.uint64)
    lane_bytes_sum = np.zeros(16, dtype=np.uint64)
    first_row = 0
    for k, sg in enumerate(segs):
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=8, credits=rows[k], quantum=chunk, total_bytes=per_conn * piece, chunk_bytes=chunk,
                                             mode=ob.SCHED_RESET_OFFSETS, state=_state(piece, 0))
        assert sg["first_row"] == first_row and sg["n_rows"] == len(exp_t) and sg["epoch_bytes"] == piece
        base = (lane_end + np.uint64(127)) // np.uint64(128) * np.uint64(128)    # where the earlier segments left every lane, 128-byte aligned
        np.testing.assert_array_equal(np.array(sg["lane_base"], dtype=np.uint64), base)
        mine = got[first_row:first_row + len(exp_t)]
        for f in ("src_off", "len", "lane", "epoch"):
            np.testing.assert_array_equal(mine[f], exp_t[f], err_msg=f"segment {k}: {f}")
        np.testing.assert_array_equal(mine["win_off"], exp_t["win_off"] + base[exp_t["lane"]], err_msg=f"segment {k}: win_off")
        np.testing.assert_array_equal(mine["tile_base"], exp_t["tile_base"] + first_row * tiles_per_chunk, err_msg=f"segment {k}: tile_base")
        used = exp_h["lane_chunks"] > 0
        lane_end[used] = base[used] + exp_h["lane_bytes"][used]
        lane_bytes_sum += exp_h["lane_bytes"]
        first_row += len(exp_t)
    np.testing.assert_array_equal(hdr["lane_bytes"], lane_bytes_sum)
    assert int(hdr["n_chunks"]) == first_row and int(hdr["total_bytes"]) == n_conn * per_conn * piece
    for q in sreqs:
        net.wait(q)
    for q in rreqs:
        assert net.wait(q) == piece
    for c in conns:
        np.testing.assert_array_equal(c["dst"].cpu().numpy(), c["src_np"])
        assert net.launch_stats(c["s"]) == {"launches": 2, "batched_requests": per_conn}
        _close(net, c)


def test_interleaved_connections_fill_launches_segment_by_segment(net):
    """Sends of three connections arriving in turn: every send opens a segment (the connection changes), eight segments fill a
    launch, and a connection's later segments carry on from where its earlier ones of the same launch left its epoch."""
    import torch
    chunk = 32 << 10
    net.reconfigure(NCCL_FUSELINK_LANES=5, NCCL_FUSELINK_CHUNKSIZE=chunk, NCCL_FUSELINK_BATCH=32, NCCL_FUSELINK_REFRESH_BATCH=64)
    net.set_credits([2, 1, 0, 3, 1])
    rng = np.random.default_rng(515)
    n_conn, per_conn = 3, 7
    sizes = [[int(rng.integers(1, 5)) * chunk - (int(rng.integers(1, chunk)) if rng.random() < 0.4 else 0) for _ in range(per_conn)] for _ in range(n_conn)]
    conns = []
    for k in range(n_conn):
        total = sum(sizes[k]) + chunk
        src_np = rng.integers(0, 256, size=total, dtype=np.uint8)
        c = _open(net, k, torch.from_numpy(src_np).cuda(), torch.zeros(total, dtype=torch.uint8, device="cuda"))
        c["src_np"] = src_np
        _send_recv(net, c["s"], c["r"], c["src"], c["dst"], chunk, 99, c["smh"], c["rmh"], src_off=sum(sizes[k]), dst_off=sum(sizes[k]))
        conns.append(c)
    rreqs, sreqs = [], []
    for q in range(per_conn):
        for k, c in enumerate(conns):
            off = sum(sizes[k][:q])
            rc, req = net.irecv(c["r"], [c["dst"].data_ptr() + off], [sizes[k][q]], [q], [c["rmh"]])
            assert rc == 0 and req
            rreqs.append((req, sizes[k][q]))
    for q in range(per_conn):
        for k, c in enumerate(conns):
            off = sum(sizes[k][:q])
            rc, req = net.isend(c["s"], c["src"].data_ptr() + off, sizes[k][q], q, c["smh"])
            assert rc == 0 and req
            sreqs.append(req)
    net.flush(conns[0]["s"])
    segs, got, hdr = net.last_launch(conns[0]["s"])
    assert 1 <= len(segs) <= 8
    for q in sreqs:
        net.wait(q)
    for q, n in rreqs:
        assert net.wait(q) == n
    launches = 0
    for c in conns:
        np.testing.assert_array_equal(c["dst"].cpu().numpy(), c["src_np"])
        launches = max(launches, net.launch_stats(c["s"])["launches"])
        _close(net, c)
    assert launches <= 1 + 3      # 21 sends, eight segments to a launch: three launches behind the warm-up


def test_more_connections_than_a_pool_of_their_own_windows_would_allow(net):
    """Every connection that stages on a GPU shares that GPU's lane windows (src/fuselink.h:271-272), so the number of
    connections is not bounded by the unit pool: twelve connections at 8 lanes x 4 units would need 384 units of the
    reference's 256 (src/cumem.cu:9) if each bound its own."""
    import torch
    net.reconfigure(NCCL_FUSELINK_LANES=8, NCCL_FUSELINK_CHUNKSIZE=64 << 10)
    rng = np.random.default_rng(12)
    size = 1 << 20
    conns = []
    for k in range(12):
        src_np = rng.integers(0, 256, size=size, dtype=np.uint8)
        c = _open(net, k % 8, torch.from_numpy(src_np).cuda(), torch.zeros(size, dtype=torch.uint8, device="cuda"))
        c["src_np"] = src_np
        conns.append(c)
    reqs = []
    for k, c in enumerate(conns):
        rc, rreq = net.irecv(c["r"], [c["dst"].data_ptr()], [size], [k], [c["rmh"]])
        assert rc == 0 and rreq
        rc, sreq = net.isend(c["s"], c["src"].data_ptr(), size, k, c["smh"])
        assert rc == 0 and sreq
        reqs.append((sreq, rreq))
    for sreq, rreq in reqs:
        net.wait(sreq)
        assert net.wait(rreq) == size
    for c in conns:
        np.testing.assert_array_equal(c["dst"].cpu().numpy(), c["src_np"])
        _close(net, c)


@pytest.mark.parametrize("block", range(4))
def test_random_request_streams(net, block):
    """Seeded random connections: lanes, chunk size, batching, refresh cadence, window size, QP split, policy,
    request sizes (whole chunks or arbitrary, zero included) and the interleaving of irecv / isend / test all
    vary; every byte must arrive, nothing may be written past the last request."""
    import torch
    buf_bytes = 24 << 20
    src = torch.randint(0, 255, (buf_bytes,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros_like(src)
    for seed in range(block * 12, block * 12 + 12):
        rng = np.random.default_rng(600_000 + seed)
        lanes = int(rng.integers(1, 17))
        chunk = int(rng.choice([4096, 65536, 256 << 10, 512 << 10, 100 * 128]))
        env = dict(NCCL_FUSELINK_LANES=lanes, NCCL_FUSELINK_CHUNKSIZE=chunk, NCCL_FUSELINK_BATCH=int(rng.choice([1, 2, 8])),
                   NCCL_FUSELINK_REFRESH_BATCH=int(rng.choice([1, 3, 8])), NCCL_FUSELINK_WINDOW_UNITS=int(rng.choice([1, 2, 4])),
                   NCCL_IB_QPS_PER_CONNECTION=int(rng.choice([1, 1, 3])), NCCL_FUSELINK_POLICY=int(rng.choice([0, 1, 1])))
        net.reconfigure(**env)
        net.set_credits([int(c) for c in rng.integers(0, 9, size=lanes)] if rng.random() < 0.8 else [])
        dst.zero_()
        lcomm, s, r = net.connect_pair(int(rng.integers(0, lanes)))
        _, smh = net.regMr(s, src.data_ptr(), buf_bytes, P.NCCL_PTR_CUDA)
        _, rmh = net.regMr(r, dst.data_ptr(), buf_bytes, P.NCCL_PTR_CUDA)
        n_req = int(rng.integers(1, 30))
        if rng.random() < 0.5:
            sizes = [int(rng.integers(1, 9)) * chunk for _ in range(n_req)]
        else:
            sizes = [int(rng.integers(0, 1 << 20)) for _ in range(n_req)]
        while sum(sizes) > buf_bytes:
            sizes.pop()
        n_req = len(sizes)
        offs = np.concatenate([[0], np.cumsum(sizes)[:-1]]).astype(np.int64)
        inflight_max = int(rng.integers(1, 9))
        posted = sent = done_r = done_s = spins = 0
        rq, sq = [], []
        while done_r < n_req or done_s < n_req:
            spins += 1
            assert spins < 2_000_000, f"seed {seed}: no progress"
            if posted < n_req and posted - done_r < inflight_max:
                rc, q = net.irecv(r, [dst.data_ptr() + int(offs[posted])], [sizes[posted]], [posted], [rmh])
                assert rc == 0
                if q:
                    rq.append((q, sizes[posted]))
                    posted += 1
            if sent < posted and rng.random() < 0.7:
                rc, q = net.isend(s, src.data_ptr() + int(offs[sent]), sizes[sent], sent, smh)
                assert rc == 0
                if q:
                    sq.append(q)
                    sent += 1
            if rq and rng.random() < 0.5:
                rc, d, sz = net.test(rq[0][0])
                assert rc == 0
                if d:
                    assert sz == rq[0][1]
                    rq.pop(0)
                    done_r += 1
            if sq and rng.random() < 0.5:
                rc, d, _ = net.test(sq[0])
                assert rc == 0
                if d:
                    sq.pop(0)
                    done_s += 1
        torch.cuda.synchronize()
        tot = int(sum(sizes))
        assert torch.equal(dst[:tot], src[:tot]), f"seed {seed}: data differs ({env})"
        assert not dst[tot:tot + 4096].any(), f"seed {seed}: wrote past the end"
        net.deregMr(s, smh), net.deregMr(r, rmh)
        net.closeSend(s), net.closeRecv(r), net.closeListen(lcomm)


@pytest.mark.parametrize("name", ["fuselink", "libnccl-net-fuselink.so"])
def test_rccl_loads_the_plugin_and_probes_every_device(name):
    """What the reference's README asks of a user (NCCL_NET_PLUGIN=fuselink, README.md:35-40), under this
    image's RCCL: the library is found by name, its v8 table is taken, init / devices / getProperties run,
    and RCCL's GPU Direct check registers device memory through a connection it opens on every virtual NIC."""
    import os
    import subprocess
    import sys

    from fuselink_amd import build
    libdir = os.path.dirname(build.lib_path())
    if name == "fuselink" and not os.path.exists(os.path.join(libdir, "librccl-net-fuselink.so")):
        pytest.skip("librccl-net-fuselink.so (RCCL's name for the plugin) not built")
    env = dict(os.environ, NCCL_NET_PLUGIN=name, NCCL_DEBUG="INFO", NCCL_DEBUG_SUBSYS="INIT,NET",
               LD_LIBRARY_PATH=libdir + ":" + os.environ.get("LD_LIBRARY_PATH", ""), MASTER_PORT="29541")
    probe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rccl_probe.py")
    res = subprocess.run([sys.executable, probe], capture_output=True, text=True, timeout=170, env=env)
    log = res.stdout + res.stderr
    assert res.returncode == 0, log[-3000:]
    assert "Loaded net plugin FuseLink (v8)" in log, log[-3000:]
    assert "Using network FuseLink" in log
    assert "NET/FuseLink : 8 lanes" in log          # the plugin's own init line, through RCCL's logger
    for dev in range(8):
        assert f"'fuselink{dev}'" in log           # getProperties of every virtual NIC was read
    assert "allreduce 1024.0" in log


_SEED0 = int(__import__("os").environ.get("FUSELINK_RANDOM_SEED_FIRST", "0"))


@pytest.mark.parametrize("seed", range(_SEED0, _SEED0 + int(__import__("os").environ.get("FUSELINK_RANDOM_SEEDS", "10"))))
def test_random_traffic_of_several_connections_arrives_intact(net, seed):
    """Random mixes of what the paths distinguish: 1 to 5 connections on one GPU; requests of 0 bytes, a few bytes, ragged
    lengths, whole chunks, more than the engine takes (launch pairs), more than the windows hold (waves); receives
    larger than their sends; credit rows that change between refreshes; every completion mode with and without the
    engine.  One thread posts and polls in random order, as several proxy threads' calls could interleave.  Every
    destination byte is compared with the source (the rest must stay zero) and every receive reports its send's size."""
    import torch
    rng = np.random.default_rng(9100 + seed)
    lanes = int(rng.choice([1, 2, 3, 5, 8, 16]))
    chunk = int(rng.choice([4 << 10, 32 << 10, 64 << 10, 256 << 10]))
    completion, engine = [(2, 1), (2, 1), (2, 0), (1, 0), (0, 0)][seed % 5]
    cadence = int(rng.choice([2, 8, 1000]))
    net.reconfigure(NCCL_FUSELINK_LANES=lanes, NCCL_FUSELINK_CHUNKSIZE=chunk, NCCL_FUSELINK_WINDOW_UNITS=int(rng.choice([1, 2, 4])),
                    NCCL_FUSELINK_REFRESH_BATCH=cadence, NCCL_FUSELINK_COMPLETION=completion, NCCL_FUSELINK_ENGINE=engine,
                    NCCL_FUSELINK_ENGINE_SETS=int(rng.choice([1, 2, 3])), NCCL_FUSELINK_BATCH=int(rng.choice([2, 8, 32])),
                    NCCL_FUSELINK_ONE_PASS=int(__import__("os").environ.get("FUSELINK_RANDOM_ONE_PASS", seed % 3 != 2)))
    net.set_credits([int(c) for c in rng.integers(0, 5, size=lanes)])

    def draw_size():
        kind = rng.integers(0, 8)
        if kind == 0:
            return 0
        if kind == 1:
            return int(rng.integers(1, 200))
        if kind == 2:
            return int(rng.integers(1, 4 * chunk))                       # ragged
        if kind == 3:
            return int(rng.integers(1, 9)) * chunk                      # whole chunks
        if kind == 4:
            return int(rng.integers(1, 9)) * chunk + int(rng.integers(1, chunk))
        if kind == 5:
            return (1 << 20) + int(rng.integers(1, 1 << 20))             # past what the engine takes
        if kind == 6:
            return int(rng.integers(1, 3)) * (6 << 20) + int(rng.integers(0, 4097))   # more than small windows hold
        return 512 << 10

    n_conn = int(rng.integers(1, 6))
    conns = []
    for k in range(n_conn):
        sizes = [draw_size() for _ in range(int(rng.integers(4, 25)))]
        slack = [int(rng.integers(0, 300)) if rng.random() < 0.3 else 0 for _ in sizes]     # the receive may be larger than the send
        offs = np.concatenate([[0], np.cumsum([s + e + int(rng.integers(0, 3)) * 7 for s, e in zip(sizes, slack)])]).astype(np.int64)
        total = int(offs[-1]) + 64
        src_np = rng.integers(1, 256, size=total, dtype=np.uint8)       # no zero byte: an unwritten destination byte shows
        c = _open(net, k % lanes, torch.from_numpy(src_np).cuda(), torch.zeros(total, dtype=torch.uint8, device="cuda"))
        c.update(src_np=src_np, sizes=sizes, slack=slack, offs=offs, posted=0, sent=0, rq=[], sq=[], window=int(rng.integers(1, 9)))
        conns.append(c)
    steps = 0
    while any(c["sent"] < len(c["sizes"]) or c["rq"] or c["sq"] for c in conns):
        steps += 1
        assert steps < 2_000_000, "no progress"
        c = conns[int(rng.integers(0, n_conn))]
        act = rng.integers(0, 4)
        if act == 0 and c["posted"] < len(c["sizes"]) and len(c["rq"]) < c["window"]:
            q = c["posted"]
            rc, req = net.irecv(c["r"], [c["dst"].data_ptr() + int(c["offs"][q])], [c["sizes"][q] + c["slack"][q]], [q], [c["rmh"]])
            assert rc == 0
            if req:                                                        # none: the refresh gate holds it until the receives in flight are done
                c["rq"].append((req, c["sizes"][q]))
                c["posted"] += 1
        elif act == 1 and c["sent"] < c["posted"]:
            q = c["sent"]
            rc, req = net.isend(c["s"], c["src"].data_ptr() + int(c["offs"][q]), c["sizes"][q], q, c["smh"])
            assert rc == 0 and req
            c["sq"].append(req)
            c["sent"] += 1
        elif act == 2 and c["rq"]:
            rc, done, got = net.test(c["rq"][0][0])
            assert rc == 0
            if done:
                assert got == c["rq"][0][1]
                c["rq"].pop(0)
        elif act == 3 and c["sq"]:
            rc, done, _ = net.test(c["sq"][0])
            assert rc == 0
            if done:
                c["sq"].pop(0)
        if rng.random() < 0.002:
            net.set_credits([int(x) for x in rng.integers(0, 5, size=lanes)])   # taken up at the connections' next refresh
    for c in conns:
        exp = np.zeros_like(c["src_np"])
        for q, n in enumerate(c["sizes"]):
            o = int(c["offs"][q])
            exp[o:o + n] = c["src_np"][o:o + n]
        got = c["dst"].cpu().numpy()
        if not np.array_equal(got, exp):    # say where: which request, which of its bytes, what lies there instead
            bad = np.flatnonzero(got != exp)
            runs = np.split(bad, np.flatnonzero(np.diff(bad) > 1) + 1)
            q = int(np.searchsorted(c["offs"], bad[0], side="right")) - 1
            raise AssertionError(f"seed {seed}: lanes {lanes} chunk {chunk} completion {completion} engine {engine}; connection {conns.index(c)} of {n_conn}: "
                                 f"{bad.size} bytes differ in {len(runs)} runs, the first [{bad[0]}, {runs[0][-1] + 1}) = request {q} (size {c['sizes'][q]}, "
                                 f"at {int(c['offs'][q])}) + {bad[0] - int(c['offs'][q])}; sizes {c['sizes']}; got {got[bad[0]:bad[0] + 8].tolist()} "
                                 f"expected {exp[bad[0]:bad[0] + 8].tolist()}; runs {[(int(r[0]), int(r.size)) for r in runs[:8]]}")
        _close(net, c)


def test_an_engine_that_goes_down_fails_its_requests_and_traffic_falls_back_to_launches(net):
    """The lane engine's waits are bounded; when one runs out the engine reports it and goes down.  A healthy GPU misses no
    two-second limit, so the condition is forced from the host: an engine started while flh_tune("engine_inject_fault")
    is set reports the failure in place of executing its first batch, and every workgroup leaves.  The requests the
    engine held complete with ncclRemoteError (as a queue pair in the error state completes its work requests,
    src/plugin.cc:1839-1861) and are freed, nothing hangs, and later requests of the same connection -- across its next
    refresh boundaries, on the default cadence of 8 -- and of a connection opened afterwards move their bytes through
    launch pairs."""
    import ctypes as C
    import time
    import torch
    piece = 512 << 10
    net.reconfigure(NCCL_FUSELINK_LANES=8, NCCL_FUSELINK_CHUNKSIZE=256 << 10, NCCL_FUSELINK_BATCH=8, NCCL_FUSELINK_ENGINE=1)
    net.lib.flh_tune.argtypes = [C.c_char_p, C.c_int64]
    rng = np.random.default_rng(77)
    n, later = 32, 20
    src_np = rng.integers(1, 256, size=(n + 1 + later) * piece, dtype=np.uint8)
    c = _open(net, 0, torch.from_numpy(src_np).cuda(), torch.zeros((n + 1 + later) * piece, dtype=torch.uint8, device="cuda"))
    # one request on its own passes through the engine and takes the connection off its refresh boundary
    _send_recv(net, c["s"], c["r"], c["src"], c["dst"], piece, 99, c["smh"], c["rmh"], src_off=n * piece, dst_off=n * piece)
    time.sleep(0.05)         # far beyond the engine's idle limit: it has gone down, the next batch starts it again
    assert net.lib.flh_tune(b"engine_inject_fault", 1) == 0
    try:
        reqs = []
        for q in range(n):
            rc, rreq = net.irecv(c["r"], [c["dst"].data_ptr() + q * piece], [piece], [q], [c["rmh"]])
            assert rc == 0 and rreq
            reqs.append(rreq)
        for q in range(n):   # every eighth send fills a batch, which goes out inside that isend
            rc, sreq = net.isend(c["s"], c["src"].data_ptr() + q * piece, piece, q, c["smh"])
            assert rc == 0 and sreq
            reqs.append(sreq)
        failed = finished = 0
        deadline = time.time() + 20
        pending = list(reqs)
        while pending:
            assert time.time() < deadline, "requests neither completed nor failed"
            rc, done, _ = net.test(pending[0])
            if rc != 0:
                assert rc == P.ncclRemoteError
                failed += 1
                pending.pop(0)
            elif done:
                finished += 1
                pending.pop(0)
    finally:
        assert net.lib.flh_tune(b"engine_inject_fault", 0) == 0
    # the first batch's eight sends and eight receives at least; what was sent after the failure showed went by launches
    assert failed >= 16 and finished + failed == 2 * n
    # every request, failed or not, has been freed and counted: the connection's next refreshes (at 40 and 48 completed
    # receives) are not held back, and its later traffic goes by launch pairs and arrives
    assert net.free_requests(c["s"]) == 256 and net.free_requests(c["r"]) == 256
    st = net.comm_stats(c["r"])
    assert st["n_finished"] == n + 1 and st["in_flight"] == 0
    for q in range(n + 1, n + 1 + later):
        rreq, deadline = None, time.time() + 10
        while not rreq:
            rc, rreq = net.irecv(c["r"], [c["dst"].data_ptr() + q * piece], [piece], [q], [c["rmh"]])
            assert rc == 0 and time.time() < deadline, "a later receive was never accepted: the connection stalled at its refresh"
        rc, sreq = net.isend(c["s"], c["src"].data_ptr() + q * piece, piece, q, c["smh"])
        assert rc == 0 and sreq
        net.wait(sreq)
        assert net.wait(rreq) == piece
    np.testing.assert_array_equal(c["dst"].cpu().numpy()[(n + 1) * piece:], src_np[(n + 1) * piece:])
    assert net.comm_stats(c["r"])["refreshes"] >= 3
    # the GPU's staging side lives on: new traffic goes by launch pairs and arrives
    src2_np = rng.integers(0, 256, size=4 * piece, dtype=np.uint8)
    c2 = _open(net, 1, torch.from_numpy(src2_np).cuda(), torch.zeros(4 * piece, dtype=torch.uint8, device="cuda"))
    for q in range(4):
        _send_recv(net, c2["s"], c2["r"], c2["src"], c2["dst"], piece, q, c2["smh"], c2["rmh"], src_off=q * piece, dst_off=q * piece)
    np.testing.assert_array_equal(c2["dst"].cpu().numpy(), src2_np)
    assert net.launch_stats(c2["s"])["launches"] >= 1
    _close(net, c2)
    _close(net, c)
