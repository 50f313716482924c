"""flh_schedule_static -- the scheduler entry point that allocates nothing (its scan over several workgroups uses a
static per-device workspace of the library's own) -- against flh_schedule with a lent workspace, bit for bit, and
against the CPU oracle: two calls in a row on the same GPU, the second with a shorter chunk list, so that what the
first call left in the shared workspace must not leak into the second."""
import ctypes as C

import numpy as np
import pytest

from tests import oracle_binding as ob

pytestmark = pytest.mark.gpu


def _dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _run(core, torch, *, static, sizes, credits, lanes, quantum, epoch_len, tile, state_np):
    d_state = _dev(torch, np.array([state_np], dtype=ob.STATE_DTYPE).view(np.uint8))
    sched = core.schedule(n_lanes=lanes, credits=_dev(torch, credits.view(np.int32)), quantum=quantum,
                          sizes=_dev(torch, sizes.view(np.int32)), epoch_len=epoch_len, tile_bytes=tile, state=d_state,
                          workspace=not static, static_workspace=static)
    torch.cuda.synchronize()
    return sched.table_numpy(), sched.hdr_numpy(), core.state_numpy(d_state)


def test_static_workspace_scheduler_equals_lent_workspace_twice_in_a_row():
    import torch

    from fuselink_amd import core
    core.init(0)
    rng = np.random.default_rng(90210)
    lanes, quantum, epoch_len, tile = 11, 4096, 1000, 4096
    credits = rng.integers(0, 7, size=(4, lanes)).astype(np.uint32)
    credits[2, :] = 0                                   # a row without credit: the static policy stands in
    state = np.zeros(1, dtype=ob.STATE_DTYPE)[0]
    state["epoch_bytes"], state["chunk_index"] = 12345, 777
    state["lane_off"][:lanes] = rng.integers(0, 1 << 28, size=lanes)
    for n in (20000, 5000):                             # both long enough for the scan over several workgroups (>= 4096)
        sizes = rng.integers(0, 9000, size=n).astype(np.uint32)
        kw = dict(sizes=sizes, credits=credits, lanes=lanes, quantum=quantum, epoch_len=epoch_len, tile=tile, state_np=state)
        lent_t, lent_h, lent_s = _run(core, torch, static=False, **kw)
        got_t, got_h, got_s = _run(core, torch, static=True, **kw)
        exp_t, exp_h, exp_s = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=quantum, sizes=sizes, epoch_len=epoch_len,
                                                 tile_bytes=tile, state=state)
        for f in ob.DESC_DTYPE.names:
            np.testing.assert_array_equal(got_t[f], lent_t[f], err_msg=f"n={n}: table field {f} differs from flh_schedule's")
            np.testing.assert_array_equal(got_t[f], exp_t[f], err_msg=f"n={n}: table field {f} differs from the oracle's")
        for f in ("total_bytes", "total_tiles", "n_chunks", "flags", "uniform_tiles", "lane_bytes", "lane_chunks"):
            np.testing.assert_array_equal(got_h[f], lent_h[f], err_msg=f"n={n}: header field {f}")
            np.testing.assert_array_equal(got_h[f], exp_h[f], err_msg=f"n={n}: header field {f} (oracle)")
        for f in ob.STATE_DTYPE.names:
            np.testing.assert_array_equal(got_s[f], lent_s[f], err_msg=f"n={n}: state field {f}")
            np.testing.assert_array_equal(got_s[f], exp_s[f], err_msg=f"n={n}: state field {f} (oracle)")
        state = got_s                                   # the second call carries on from the first


def test_static_workspace_scheduler_allocates_nothing_and_replays_from_a_graph():
    """What the header promises of flh_schedule_static beyond its results: the call takes no device memory (the driver's
    count of free memory reads the same before and after a run of calls whose buffers all exist beforehand), and it can
    be recorded into a HIP graph -- a capture refuses any allocation -- and replayed with new sizes in the same buffers,
    every replay checked against the oracle, with eager work and synchronizations of the program's own in between."""
    import torch

    from fuselink_amd import _lib, core
    core.init(0)
    lib = _lib.load()
    rng = np.random.default_rng(4711)
    lanes, n, quantum, tile = 9, 12000, 2048, 4096
    credits = rng.integers(0, 6, size=(3, lanes)).astype(np.uint32)
    sizes = torch.zeros(n, dtype=torch.int32, device="cuda")
    d_credits = _dev(torch, credits.view(np.int32))
    out = core.new_schedule_buffers(n, tile_bytes=tile)
    p = _lib.SchedParams()
    p.d_sizes, p.n_chunks, p.n_lanes = sizes.data_ptr(), n, lanes
    p.d_credits, p.n_rows, p.epoch_len, p.quantum, p.tile_bytes = d_credits.data_ptr(), 3, 1000, quantum, tile
    p.d_table, p.d_hdr = out.table.data_ptr(), out.hdr.data_ptr()
    side = torch.cuda.Stream()
    s_ptr = C.c_void_p(side.cuda_stream)
    _lib.check(lib.flh_schedule_static(C.byref(p), s_ptr))      # (first call on the device: the workspace's address is resolved)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(20):
        _lib.check(lib.flh_schedule_static(C.byref(p), s_ptr))
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"device memory moved by {free_before - free_after} bytes across 20 calls"

    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _lib.check(lib.flh_schedule_static(C.byref(p), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    for rep in range(4):
        sizes_np = rng.integers(0, 5000, size=n).astype(np.uint32)
        sizes.copy_(torch.from_numpy(sizes_np.view(np.int32)))
        out.table.zero_()                                       # eager work of the program's own between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        exp_t, exp_h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits, quantum=quantum, sizes=sizes_np, epoch_len=1000, tile_bytes=tile)
        assert out.table_numpy().tobytes() == exp_t.tobytes(), f"replay {rep}"
        np.testing.assert_array_equal(out.hdr_numpy()["lane_bytes"], exp_h["lane_bytes"], err_msg=f"replay {rep}")


def test_static_workspace_scheduler_refuses_lists_beyond_its_limit():
    import torch

    from fuselink_amd import _lib, core
    core.init(0)
    n = (1 << 20) + 1
    out = core.new_schedule_buffers(16)
    p = _lib.SchedParams(None, 0, 0, None, 0, n, 2, None, 1, 0, 4096, 32768, 0, None, out.table.data_ptr(), out.hdr.data_ptr())
    p.inline_credits[0] = p.inline_credits[1] = 1
    with pytest.raises(_lib.FuseLinkError, match="exceed"):
        _lib.check(_lib.load().flh_schedule_static(C.byref(p), None))
    torch.cuda.synchronize()
