"""Host-side driver of the gfx950 data path: thin, typed wrappers over the C ABI in
include/fuselink_hip.h.  PyTorch is used only to own device memory and streams."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np
import torch

from . import _lib
from ._lib import MAX_LANES, BatchParams, ChunkDesc, SchedHdr, SchedParams, SchedState, UniformParams, Windows, check

TILE_BYTES = 32768
UNIT_BYTES = 2 * 1024 * 1024
SCHED_RESET_OFFSETS = 1
SCHED_MIRROR = 2
SCHED_NEW_EPOCH = 4
SCHED_F_NO_CREDIT = 1

DESC_DTYPE = np.dtype([("src_off", "<u8"), ("win_off", "<u8"), ("len", "<u4"), ("lane", "<u4"),
                       ("tile_base", "<u4"), ("epoch", "<u4")])
HDR_DTYPE = np.dtype([("total_bytes", "<u8"), ("total_tiles", "<u4"), ("n_chunks", "<u4"), ("flags", "<u4"),
                      ("uniform_tiles", "<u4"), ("lane_bytes", "<u8", (MAX_LANES,)), ("lane_chunks", "<u4", (MAX_LANES,))])
TILE_DESC_DTYPE = np.dtype([("src_off", "<u8"), ("win_off", "<u8"), ("len", "<u4"), ("lane", "<u4"), ("row", "<u4"), ("pad", "<u4")])
STATE_DTYPE = np.dtype([("epoch_bytes", "<u8"), ("chunk_index", "<u8"), ("lane_off", "<u8", (MAX_LANES,))])
assert DESC_DTYPE.itemsize == C.sizeof(ChunkDesc) == 32
assert HDR_DTYPE.itemsize == C.sizeof(SchedHdr)
assert STATE_DTYPE.itemsize == C.sizeof(SchedState)


def init(device: int = 0) -> None:
    check(_lib.load().flh_init(device))


def tune(key: str, value: int) -> None:
    check(_lib.load().flh_tune(key.encode(), int(value)))


PROF_KERNELS = {1: "schedule", 2: "stripe", 3: "reassemble", 4: "gather", 5: "scatter", 6: "copy", 7: "stage_deliver"}


def prof_begin(capacity: int) -> None:
    check(_lib.load().flh_prof_begin(capacity))


def prof_end(capacity: int):
    """Returns {kernel name: [durations in us]} of the launches made since prof_begin."""
    us = (C.c_double * capacity)()
    kid = (C.c_int * capacity)()
    n = check(_lib.load().flh_prof_end(us, kid, capacity))
    out = {}
    for i in range(min(n, capacity)):
        out.setdefault(PROF_KERNELS.get(kid[i], str(kid[i])), []).append(us[i])
    return out


def _stream_ptr(stream: Optional[torch.cuda.Stream]) -> C.c_void_p:
    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> C.c_void_p:
    return C.c_void_p(0 if t is None else t.data_ptr())


def _dev_bytes(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


@dataclass
class Schedule:
    """Device-resident chunk -> lane table and its summary."""
    table: torch.Tensor      # uint8 [n * 32]
    hdr: torch.Tensor        # uint8 [sizeof(flh_sched_hdr)]
    n_chunks: int
    tile_bytes: int
    table_by_lane: Optional[torch.Tensor] = None   # the same rows in destination order (uniform split only)
    tiles: Optional[torch.Tensor] = None           # uint8 [capacity * 32]: one flh_tile_desc per copy tile
    tiles_cap: int = 0
    workspace: Optional[torch.Tensor] = None       # scratch for the scan scheduler over several workgroups

    def tiles_numpy(self, n_tiles: int) -> np.ndarray:
        return self.tiles[: n_tiles * TILE_DESC_DTYPE.itemsize].cpu().numpy().view(TILE_DESC_DTYPE).copy()

    def table_numpy(self) -> np.ndarray:
        raw = self.table[: self.n_chunks * DESC_DTYPE.itemsize].cpu().numpy()
        return raw.view(DESC_DTYPE).copy()

    def hdr_numpy(self) -> np.ndarray:
        return self.hdr.cpu().numpy().view(HDR_DTYPE)[0].copy()

    def table_by_lane_numpy(self) -> np.ndarray:
        raw = self.table_by_lane[: self.n_chunks * DESC_DTYPE.itemsize].cpu().numpy()
        return raw.view(DESC_DTYPE).copy()


def new_state(device="cuda") -> torch.Tensor:
    return torch.zeros(STATE_DTYPE.itemsize, dtype=torch.uint8, device=device)


def state_numpy(state: torch.Tensor) -> np.ndarray:
    return state.cpu().numpy().view(STATE_DTYPE)[0].copy()


def schedule(*, n_lanes: int, credits: torch.Tensor, quantum: int, sizes: Optional[torch.Tensor] = None,
             total_bytes: int = 0, chunk_bytes: int = 0, src_off: Optional[torch.Tensor] = None, src_base: int = 0,
             epoch_len: int = 0, tile_bytes: int = TILE_BYTES, mode: int = 0, state: Optional[torch.Tensor] = None,
             out: Optional[Schedule] = None, stream: Optional[torch.cuda.Stream] = None, by_lane: bool = False,
             tiles_capacity: int = 0, workspace: bool = False, wave_chunks: int = 0, static_workspace: bool = False) -> Schedule:
    """Launches the scheduler kernel (flh_schedule).  `credits` is a uint32/int32 device tensor of
    shape [rows, n_lanes]; `sizes` a uint32/int32 device tensor of chunk sizes, or None for the
    uniform split of `total_bytes` by `chunk_bytes`."""
    lib = _lib.load()
    inline = None
    if not isinstance(credits, torch.Tensor):
        inline = [int(c) for c in credits]  # one row, passed by value in the launch arguments
        assert len(inline) == n_lanes
    else:
        if credits.dim() == 1:
            credits = credits.view(1, -1)
        assert credits.is_cuda and credits.dtype in (torch.int32, torch.uint32) and credits.is_contiguous()
        assert credits.shape[1] == n_lanes
    if sizes is not None:
        assert sizes.is_cuda and sizes.dtype in (torch.int32, torch.uint32) and sizes.is_contiguous()
        n = sizes.numel()
    else:
        n = (total_bytes + chunk_bytes - 1) // chunk_bytes if chunk_bytes else 0
    if src_off is not None:
        assert src_off.is_cuda and src_off.dtype in (torch.int64, torch.uint64) and src_off.numel() == n
    dev = credits.device if inline is None else torch.device("cuda", torch.cuda.current_device())
    if out is None:
        out = Schedule(_dev_bytes(n * DESC_DTYPE.itemsize, dev), _dev_bytes(HDR_DTYPE.itemsize, dev), n, tile_bytes)
    else:
        assert out.table.numel() >= n * DESC_DTYPE.itemsize
        out.n_chunks, out.tile_bytes = n, tile_bytes
    if by_lane and out.table_by_lane is None:
        out.table_by_lane = _dev_bytes(max(n, 1) * DESC_DTYPE.itemsize, dev)
    p = SchedParams(_ptr(sizes), total_bytes, chunk_bytes, _ptr(src_off), src_base, n, n_lanes,
                    _ptr(credits if inline is None else None), 1 if inline is not None else credits.shape[0], epoch_len,
                    quantum, tile_bytes, mode, _ptr(state), _ptr(out.table), _ptr(out.hdr))
    if inline is not None:
        for l, c in enumerate(inline):
            p.inline_credits[l] = c
    p.d_table_by_lane = _ptr(out.table_by_lane) if by_lane else None
    if tiles_capacity:   # per-tile descriptors for stripe / reassemble (pays for tables of many unequal rows)
        if out.tiles is None or out.tiles_cap < tiles_capacity:
            out.tiles, out.tiles_cap = _dev_bytes(tiles_capacity * TILE_DESC_DTYPE.itemsize, dev), tiles_capacity
        p.d_tiles, p.tiles_cap = _ptr(out.tiles), out.tiles_cap
    p.wave_chunks = wave_chunks
    if workspace:        # lets a long list that needs the scan be scheduled by several workgroups
        need = int(lib.flh_schedule_workspace_bytes(n))
        if out.workspace is None or out.workspace.numel() < need:
            out.workspace = _dev_bytes(need, dev)
        p.d_workspace, p.workspace_bytes = _ptr(out.workspace), out.workspace.numel()
    if static_workspace:  # the library's own per-device workspace: nothing is allocated by the call (flh_schedule_static)
        assert not workspace
        check(lib.flh_schedule_static(C.byref(p), _stream_ptr(stream)))
    else:
        check(lib.flh_schedule(C.byref(p), _stream_ptr(stream)))
    return out


def make_windows(bases: Sequence[int], caps: Sequence[int]) -> Windows:
    w = Windows()
    w.n_lanes = len(bases)
    for l, (b, c) in enumerate(zip(bases, caps)):
        w.base[l] = b
        w.cap[l] = c
    return w


def windows_from_tensors(tensors: Sequence[torch.Tensor]) -> Windows:
    return make_windows([t.data_ptr() for t in tensors], [t.numel() * t.element_size() for t in tensors])


def new_status(device="cuda") -> torch.Tensor:
    return torch.zeros(1, dtype=torch.int32, device=device)


def uniform_hint(total_bytes: int, chunk_bytes: int, tile_bytes: int = TILE_BYTES) -> SchedHdr:
    """Host copy of the header fields that follow from a uniform split alone (no device read)."""
    h = SchedHdr()
    n = (total_bytes + chunk_bytes - 1) // chunk_bytes if chunk_bytes else 0
    per = (chunk_bytes + tile_bytes - 1) // tile_bytes if n else 0
    last = total_bytes - (n - 1) * chunk_bytes if n else 0
    h.total_bytes = total_bytes
    h.n_chunks = n
    h.uniform_tiles = per
    h.total_tiles = (n - 1) * per + (last + tile_bytes - 1) // tile_bytes if n else 0
    return h


def _hint_ref(hint: Optional[SchedHdr]):
    return C.byref(hint) if hint is not None else None


def stripe(src: torch.Tensor, win: Windows, sched: Schedule, status: torch.Tensor,
           stream: Optional[torch.cuda.Stream] = None, hint: Optional[SchedHdr] = None, by_lane: bool = False) -> None:
    """flh_stripe; with by_lane the rows are taken in destination order (sched.table_by_lane)."""
    table = sched.table_by_lane if by_lane else sched.table
    if sched.tiles is not None and not by_lane:
        check(_lib.load().flh_stripe_tiles(_ptr(src), src.numel() * src.element_size(), C.byref(win), _ptr(sched.tiles), sched.tiles_cap,
                                           _ptr(sched.hdr), _hint_ref(hint), _ptr(status), _stream_ptr(stream)))
        return
    check(_lib.load().flh_stripe(_ptr(src), src.numel() * src.element_size(), C.byref(win), _ptr(table),
                                 _ptr(sched.hdr), _hint_ref(hint), sched.n_chunks, sched.tile_bytes, _ptr(status),
                                 _stream_ptr(stream)))


def reassemble(dst: torch.Tensor, win: Windows, sched: Schedule, status: torch.Tensor,
               stream: Optional[torch.cuda.Stream] = None, hint: Optional[SchedHdr] = None) -> None:
    if sched.tiles is not None:
        check(_lib.load().flh_reassemble_tiles(_ptr(dst), dst.numel() * dst.element_size(), C.byref(win), _ptr(sched.tiles), sched.tiles_cap,
                                               _ptr(sched.hdr), _hint_ref(hint), _ptr(status), _stream_ptr(stream)))
        return
    check(_lib.load().flh_reassemble(_ptr(dst), dst.numel() * dst.element_size(), C.byref(win), _ptr(sched.table),
                                     _ptr(sched.hdr), _hint_ref(hint), sched.n_chunks, sched.tile_bytes, _ptr(status),
                                     _stream_ptr(stream)))


def uniform_params(total_bytes: int, chunk_bytes: int, credits: Sequence[int], *, src_base: int = 0, epoch_bytes: int = 0,
                   tile_bytes: int = TILE_BYTES) -> UniformParams:
    u = UniformParams()
    u.total_bytes, u.src_base, u.epoch_bytes = total_bytes, src_base, epoch_bytes
    u.chunk_bytes, u.n_lanes, u.tile_bytes = chunk_bytes, len(credits), tile_bytes
    for l, c in enumerate(credits):
        u.credits[l] = int(c)
    return u


def new_schedule_buffers(n_chunks: int, tile_bytes: int = TILE_BYTES, device="cuda") -> Schedule:
    return Schedule(_dev_bytes(n_chunks * DESC_DTYPE.itemsize, device), _dev_bytes(HDR_DTYPE.itemsize, device), n_chunks, tile_bytes)


def stripe_uniform(src: torch.Tensor, win: Windows, u: UniformParams, status: torch.Tensor, out: Optional[Schedule] = None,
                   stream: Optional[torch.cuda.Stream] = None) -> None:
    """Scheduler + stripe in one launch (flh_stripe_uniform); `out` receives the table and header."""
    check(_lib.load().flh_stripe_uniform(_ptr(src), src.numel() * src.element_size(), C.byref(win), C.byref(u),
                                         _ptr(out.table) if out else None, _ptr(out.hdr) if out else None, _ptr(status),
                                         _stream_ptr(stream)))


def stage_deliver_uniform(src: torch.Tensor, dst: torch.Tensor, win: Windows, u: UniformParams, status: torch.Tensor, out: Optional[Schedule] = None,
                          stream: Optional[torch.cuda.Stream] = None) -> None:
    """flh_stage_deliver_uniform: stripe into `win` and write every tile into the same place of `dst`, in one launch."""
    check(_lib.load().flh_stage_deliver_uniform(_ptr(src), src.numel() * src.element_size(), _ptr(dst), dst.numel() * dst.element_size(), C.byref(win),
                                                C.byref(u), _ptr(out.table) if out else None, _ptr(out.hdr) if out else None, _ptr(status),
                                                _stream_ptr(stream)))


def stripe_uniform_carry(src: torch.Tensor, win: Windows, landing: Windows, u: UniformParams, status: torch.Tensor, out: Optional[Schedule] = None,
                         stream: Optional[torch.cuda.Stream] = None) -> None:
    """flh_stripe_uniform_carry: stripe into `win` and carry every staged tile on into the same place of `landing`."""
    check(_lib.load().flh_stripe_uniform_carry(_ptr(src), src.numel() * src.element_size(), C.byref(win), C.byref(landing), C.byref(u),
                                               _ptr(out.table) if out else None, _ptr(out.hdr) if out else None, _ptr(status),
                                               _stream_ptr(stream)))


def reassemble_uniform(dst: torch.Tensor, win: Windows, u: UniformParams, status: torch.Tensor,
                       stream: Optional[torch.cuda.Stream] = None) -> None:
    check(_lib.load().flh_reassemble_uniform(_ptr(dst), dst.numel() * dst.element_size(), C.byref(win), C.byref(u),
                                             _ptr(status), _stream_ptr(stream)))


def batch_params(srcs: Sequence[torch.Tensor], dsts: Sequence[torch.Tensor], chunk_bytes: int, credits: Sequence[int], *,
                 epoch_bytes: int = 0, tile_bytes: int = TILE_BYTES, segments=None) -> BatchParams:
    """Several requests in one launch (flh_stripe_batch / flh_reassemble_batch).  Without `segments` they form one
    message under `credits` / `epoch_bytes`; with it, `segments` is a list of (n_req, credits, epoch_bytes), each
    scheduled as a message of its own."""
    b = BatchParams()
    sizes = [t.numel() * t.element_size() for t in srcs]
    b.u = uniform_params(sum(sizes), chunk_bytes, credits, epoch_bytes=epoch_bytes, tile_bytes=tile_bytes)
    b.n_req = len(srcs)
    for q, (s, d, n) in enumerate(zip(srcs, dsts, sizes)):
        b.d_src[q], b.d_dst[q], b.bytes[q] = s.data_ptr(), d.data_ptr(), n
    if segments is not None:
        b.n_seg = len(segments)
        for k, (n_req, row, eb) in enumerate(segments):
            b.seg[k].n_req, b.seg[k].epoch_bytes = n_req, eb
            for l, c in enumerate(row):
                b.seg[k].credits[l] = int(c)
    return b


def batch_layout(b: BatchParams):
    """flh_batch_layout: where the batch leaves every lane's window, and every segment's lane bases."""
    ends = (C.c_uint64 * MAX_LANES)()
    bases = (C.c_uint64 * (8 * MAX_LANES))()
    check(_lib.load().flh_batch_layout(C.byref(b), ends, bases))
    return list(ends), [list(bases[k * MAX_LANES:(k + 1) * MAX_LANES]) for k in range(8)]


def stripe_batch(b: BatchParams, win: Windows, status: torch.Tensor, out: Optional[Schedule] = None,
                 stream: Optional[torch.cuda.Stream] = None) -> None:
    check(_lib.load().flh_stripe_batch(C.byref(b), C.byref(win), _ptr(out.table) if out else None,
                                       _ptr(out.hdr) if out else None, _ptr(status), _stream_ptr(stream)))


def reassemble_batch(b: BatchParams, win: Windows, status: torch.Tensor, stream: Optional[torch.cuda.Stream] = None) -> None:
    check(_lib.load().flh_reassemble_batch(C.byref(b), C.byref(win), _ptr(status), _stream_ptr(stream)))


def gather_pages(pool: torch.Tensor, page_table: torch.Tensor, page_bytes: int, pages_per_chunk: int, win: Windows,
                 sched: Schedule, status: torch.Tensor, use_lds: bool = False,
                 stream: Optional[torch.cuda.Stream] = None, by_lane: bool = False) -> None:
    nbytes = pool.numel() * pool.element_size()
    check(_lib.load().flh_gather_pages(_ptr(pool), nbytes // page_bytes, _ptr(page_table), page_bytes, pages_per_chunk,
                                       C.byref(win), _ptr(sched.table_by_lane if by_lane else sched.table), sched.n_chunks, int(use_lds), _ptr(status),
                                       _stream_ptr(stream)))


def scatter_pages(pool: torch.Tensor, page_table: torch.Tensor, page_bytes: int, pages_per_chunk: int, win: Windows,
                  sched: Schedule, status: torch.Tensor, use_lds: bool = False,
                  stream: Optional[torch.cuda.Stream] = None) -> None:
    nbytes = pool.numel() * pool.element_size()
    check(_lib.load().flh_scatter_pages(_ptr(pool), nbytes // page_bytes, _ptr(page_table), page_bytes, pages_per_chunk,
                                        C.byref(win), _ptr(sched.table), sched.n_chunks, int(use_lds), _ptr(status),
                                        _stream_ptr(stream)))


def gather_pages_uniform(pool: torch.Tensor, page_table: torch.Tensor, page_bytes: int, win: Windows, u: UniformParams,
                         status: torch.Tensor, out: Optional[Schedule] = None, stream: Optional[torch.cuda.Stream] = None) -> None:
    """Scheduler + page gather in one launch (flh_gather_pages_uniform); `out` receives the table and header."""
    nbytes = pool.numel() * pool.element_size()
    check(_lib.load().flh_gather_pages_uniform(_ptr(pool), nbytes // page_bytes, _ptr(page_table), page_bytes, C.byref(win), C.byref(u),
                                               _ptr(out.table) if out else None, _ptr(out.hdr) if out else None, _ptr(status),
                                               _stream_ptr(stream)))


def scatter_pages_uniform(pool: torch.Tensor, page_table: torch.Tensor, page_bytes: int, win: Windows, u: UniformParams,
                          status: torch.Tensor, stream: Optional[torch.cuda.Stream] = None) -> None:
    nbytes = pool.numel() * pool.element_size()
    check(_lib.load().flh_scatter_pages_uniform(_ptr(pool), nbytes // page_bytes, _ptr(page_table), page_bytes, C.byref(win), C.byref(u),
                                                _ptr(status), _stream_ptr(stream)))


def copy(dst: torch.Tensor, src: torch.Tensor, stream: Optional[torch.cuda.Stream] = None) -> None:
    nbytes = src.numel() * src.element_size()
    assert dst.numel() * dst.element_size() >= nbytes
    check(_lib.load().flh_copy(_ptr(dst), _ptr(src), nbytes, _stream_ptr(stream)))


def copy_runs(dsts, srcs, nbytes, stream: Optional[torch.cuda.Stream] = None) -> None:
    """Up to 16 independent runs in one launch: run r moves nbytes[r] bytes from srcs[r] to dsts[r] (None for an empty run)."""
    n = len(nbytes)
    d = (C.c_void_p * n)(*[_ptr(t) if t is not None else None for t in dsts])
    s = (C.c_void_p * n)(*[_ptr(t) if t is not None else None for t in srcs])
    b = (C.c_uint64 * n)(*nbytes)
    check(_lib.load().flh_copy_runs(d, s, b, n, _stream_ptr(stream)))


def qp_split(size: int, nqps: int):
    off = (C.c_int * nqps)()
    ln = (C.c_int * nqps)()
    stride = check(_lib.load().flh_qp_split(size, nqps, off, ln))
    return stride, list(off), list(ln)


class Pool:
    """HIP-VMM pool of 2 MiB staging units (flh_pool_*)."""

    def __init__(self, device: int = 0, units: int = 256):
        self._h = C.c_void_p()
        check(_lib.load().flh_pool_create(device, units, C.byref(self._h)))
        self.units = units

    @property
    def handle(self) -> C.c_void_p:
        return self._h

    def free_units(self) -> int:
        return check(_lib.load().flh_pool_free_units(self._h))

    def granularity(self) -> int:
        return int(_lib.load().flh_pool_granularity(self._h))

    def slot_of(self, va: int) -> int:
        return check(_lib.load().flh_pool_slot_of(self._h, C.c_void_p(va)))

    def destroy(self) -> None:
        if self._h:
            check(_lib.load().flh_pool_destroy(self._h))
            self._h = C.c_void_p()


class Window:
    """One lane's staging window: reserved VA whose leading units are bound to pool slots."""

    def __init__(self, pool: Pool, va_bytes: int):
        self._h = C.c_void_p()
        self.pool = pool
        check(_lib.load().flh_window_create(pool.handle, va_bytes, C.byref(self._h)))

    def bind(self, nbytes: int) -> None:
        check(_lib.load().flh_window_bind(self._h, nbytes))

    def trim(self, nbytes: int) -> None:
        check(_lib.load().flh_window_trim(self._h, nbytes))

    @property
    def base(self) -> int:
        return int(_lib.load().flh_window_base(self._h) or 0)

    @property
    def bound_bytes(self) -> int:
        return int(_lib.load().flh_window_bound_bytes(self._h))

    def slots(self):
        buf = (C.c_int * 4096)()
        n = check(_lib.load().flh_window_slots(self._h, buf, 4096))
        return list(buf[: min(n, 4096)])

    def export_dmabuf(self, offset: int, nbytes: int) -> int:
        """DMA-BUF descriptor for part of the bound window (the caller closes it)."""
        fd = C.c_int(-1)
        check(_lib.load().flh_window_export_dmabuf(self._h, offset, nbytes, C.byref(fd)))
        return fd.value

    def destroy(self) -> None:
        if self._h:
            check(_lib.load().flh_window_destroy(self._h))
            self._h = C.c_void_p()


class Region:
    """regMr-time object: one window per lane for one user allocation, shared by base address."""

    def __init__(self, pool: Pool, base: int, nbytes: int, n_lanes: int, bound_bytes_per_lane: int):
        self._h = C.c_void_p()
        check(_lib.load().flh_region_acquire(pool.handle, C.c_void_p(base), nbytes, n_lanes, bound_bytes_per_lane,
                                             C.byref(self._h)))

    @property
    def handle_value(self) -> int:
        return int(self._h.value or 0)

    def refs(self) -> int:
        return check(_lib.load().flh_region_refs(self._h))

    def windows(self) -> Windows:
        w = Windows()
        check(_lib.load().flh_region_windows(self._h, C.byref(w)))
        return w

    def translate(self, lane: int, data: int) -> int:
        return int(_lib.load().flh_region_translate(self._h, lane, C.c_void_p(data)) or 0)

    def release(self) -> int:
        left = check(_lib.load().flh_region_release(self._h))
        self._h = C.c_void_p()
        return left


def read_window(base: int, nbytes: int, device="cuda") -> torch.Tensor:
    """Copies `nbytes` at device address `base` into a fresh uint8 tensor (test helper)."""
    out = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
    if nbytes:
        check(_lib.load().flh_copy(C.c_void_p(out.data_ptr()), C.c_void_p(base), nbytes, _stream_ptr(None)))
    return out[:nbytes]
