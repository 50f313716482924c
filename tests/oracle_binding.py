"""ctypes binding of the CPU oracle (oracle/libfl_oracle.so).  Test infrastructure: only tests,
the smoke check and the benchmark's CPU-baseline leg may import this."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
MAX_LANES = 16

DESC_DTYPE = np.dtype([("src_off", "<u8"), ("win_off", "<u8"), ("len", "<u4"), ("lane", "<u4"),
                       ("tile_base", "<u4"), ("epoch", "<u4")])
HDR_DTYPE = np.dtype([("total_bytes", "<u8"), ("total_tiles", "<u4"), ("n_chunks", "<u4"), ("flags", "<u4"),
                      ("uniform_tiles", "<u4"), ("lane_bytes", "<u8", (MAX_LANES,)), ("lane_chunks", "<u4", (MAX_LANES,))])
STATE_DTYPE = np.dtype([("epoch_bytes", "<u8"), ("chunk_index", "<u8"), ("lane_off", "<u8", (MAX_LANES,))])

SCHED_RESET_OFFSETS = 1
SCHED_MIRROR = 2


class Monitor(C.Structure):
    _fields_ = [("tx_status", C.c_int32 * 16), ("rx_status", C.c_int32 * 16), ("tx_last_active", C.c_int64 * 16),
                ("rx_last_active", C.c_int64 * 16)]


class Pool(C.Structure):
    _fields_ = [("mapped", C.c_uint8 * 256), ("va", C.c_uint64 * 256)]


class RegCache(C.Structure):
    _fields_ = [("base", C.c_uint64 * 64), ("nrefs", C.c_int * 64), ("n", C.c_int), ("created", C.c_int),
                ("destroyed", C.c_int)]


class ReqTab(C.Structure):
    _fields_ = [("used", C.c_uint8 * 256)]


class Fifo(C.Structure):
    _fields_ = [("idx", C.c_uint64 * 256), ("head", C.c_uint64), ("tail", C.c_uint64)]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    path = os.path.join(ORACLE_DIR, "libfl_oracle.so")
    if not os.path.exists(path):
        subprocess.run(["make", "-C", ORACLE_DIR, "libfl_oracle.so"], check=True, capture_output=True)
    L = C.CDLL(path)
    u8p, u32p, u64p, i32p, vp = (C.POINTER(C.c_uint8), C.POINTER(C.c_uint32), C.POINTER(C.c_uint64),
                                 C.POINTER(C.c_int32), C.c_void_p)
    sig = {
        "fl_split_count": (C.c_uint64, [C.c_uint64, C.c_uint32]),
        "fl_split_get": (None, [C.c_uint64, C.c_uint32, C.c_uint64, u64p, u32p]),
        "fl_step_size": (C.c_uint32, [C.c_uint64, C.c_uint32, C.c_uint32]),
        "fl_qp_split": (C.c_int, [C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
        "fl_lane_static": (C.c_int, [C.c_int, C.c_int]),
        "fl_refresh_rx_due": (C.c_int, [C.c_int64, C.c_uint64, C.c_uint64]),
        "fl_refresh_tx_due": (C.c_int, [C.c_int64]),
        "fl_mon_init": (None, [C.POINTER(Monitor)]),
        "fl_mon_mark_tx": (None, [C.POINTER(Monitor), C.c_int, C.c_int, C.c_int64]),
        "fl_mon_mark_rx": (None, [C.POINTER(Monitor), C.c_int, C.c_int, C.c_int64]),
        "fl_mon_tick": (None, [C.POINTER(Monitor), C.c_int64]),
        "fl_mon_idle_pick_tx": (C.c_int, [C.POINTER(Monitor), C.c_int]),
        "fl_mon_idle_pick_rx": (C.c_int, [C.POINTER(Monitor), C.c_int, C.c_int]),
        "fl_mon_status": (None, [C.POINTER(Monitor), C.c_int, i32p]),
        "fl_credits_from_status": (None, [i32p, C.c_int, C.c_int, C.c_uint32, u32p]),
        "fl_tx_usage_mask": (C.c_uint32, [i32p, C.c_int, C.c_int]),
        "fl_rx_credits_from_status": (None, [i32p, C.c_int, C.c_int, C.c_uint32, C.c_uint32, u32p]),
        "fl_credit_schedule": (C.c_int, [vp, C.c_uint64, C.c_uint32, vp, C.c_uint64, C.c_uint32, C.c_uint32, vp,
                                         C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint32, C.c_uint32, vp, vp, vp]),
        "fl_table_by_lane": (C.c_int, [vp, C.c_uint32, C.c_uint32, C.c_uint32, vp]),
        "fl_align_up": (C.c_uint64, [C.c_uint64, C.c_uint64]),
        "fl_window_units": (C.c_uint64, [C.c_uint64, C.c_uint64]),
        "fl_translate": (C.c_uint64, [C.c_uint64, C.c_uint64, C.c_uint64]),
        "fl_relay_gpu": (C.c_int, [C.c_int, C.c_int, C.c_int]),
        "fl_page_span": (None, [C.c_uint64, C.c_uint64, C.c_uint64, u64p, u64p]),
        "fl_regcache_init": (None, [C.POINTER(RegCache)]),
        "fl_regcache_reg": (C.c_int, [C.POINTER(RegCache), C.c_uint64]),
        "fl_regcache_dereg": (C.c_int, [C.POINTER(RegCache), C.c_uint64]),
        "fl_pool_init": (None, [C.POINTER(Pool)]),
        "fl_pool_register": (C.c_int, [C.POINTER(Pool), C.c_uint64, C.c_uint64, C.POINTER(C.c_int), C.c_int]),
        "fl_pool_release": (C.c_int, [C.POINTER(Pool), C.c_uint64]),
        "fl_pool_lookup": (C.c_int, [C.POINTER(Pool), C.c_uint64]),
        "fl_reqtab_init": (None, [C.POINTER(ReqTab)]),
        "fl_reqtab_get": (C.c_int, [C.POINTER(ReqTab)]),
        "fl_reqtab_free": (None, [C.POINTER(ReqTab), C.c_int]),
        "fl_fifo_init": (None, [C.POINTER(Fifo)]),
        "fl_fifo_post": (C.c_int, [C.POINTER(Fifo)]),
        "fl_fifo_match": (C.c_int, [C.POINTER(Fifo)]),
        "fl_cpu_stripe": (None, [vp, vp, vp, C.c_uint32, C.c_uint32]),
        "fl_cpu_reassemble": (None, [vp, vp, vp, C.c_uint32, C.c_uint32]),
        "fl_cpu_stripe_mt": (None, [vp, vp, vp, C.c_uint32, C.c_uint32, C.c_int]),
        "fl_cpu_reassemble_mt": (None, [vp, vp, vp, C.c_uint32, C.c_uint32, C.c_int]),
        "fl_cpu_gather_pages": (None, [vp, vp, C.c_uint32, C.c_uint32, vp, vp, C.c_uint32]),
        "fl_cpu_scatter_pages": (None, [vp, vp, C.c_uint32, C.c_uint32, vp, vp, C.c_uint32]),
        "fl_cpu_baseline_run": (C.c_double, [vp, C.c_uint64, vp, vp, C.c_uint32, C.c_uint32, C.c_int, C.c_int,
                                             C.c_int, C.POINTER(C.c_double)]),
        "fl_cpu_cores": (C.c_int, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def _vp(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def split(nbytes: int, chunk: int):
    L = lib()
    n = L.fl_split_count(nbytes, chunk)
    offs, lens = [], []
    o, l = C.c_uint64(), C.c_uint32()
    for i in range(n):
        L.fl_split_get(nbytes, chunk, i, C.byref(o), C.byref(l))
        offs.append(o.value)
        lens.append(l.value)
    return offs, lens


def qp_split(size: int, nqps: int):
    off = (C.c_int * nqps)()
    ln = (C.c_int * nqps)()
    stride = lib().fl_qp_split(size, nqps, off, ln)
    return stride, list(off), list(ln)


def credit_schedule(*, n_lanes, credits, quantum, sizes=None, total_bytes=0, chunk_bytes=0, src_off=None, src_base=0,
                    epoch_len=0, tile_bytes=32768, mode=0, state=None):
    """Returns (table, hdr, state_out) as numpy structured arrays."""
    credits = np.ascontiguousarray(np.asarray(credits, dtype=np.uint32).reshape(-1, n_lanes))
    if sizes is not None:
        sizes = np.ascontiguousarray(np.asarray(sizes, dtype=np.uint32))
        n = sizes.size
    else:
        n = (total_bytes + chunk_bytes - 1) // chunk_bytes if chunk_bytes else 0
    if src_off is not None:
        src_off = np.ascontiguousarray(np.asarray(src_off, dtype=np.uint64))
    table = np.zeros(max(n, 1), dtype=DESC_DTYPE)
    hdr = np.zeros(1, dtype=HDR_DTYPE)
    st = np.zeros(1, dtype=STATE_DTYPE) if state is None else np.array([state], dtype=STATE_DTYPE)
    rc = lib().fl_credit_schedule(_vp(sizes), total_bytes, chunk_bytes, _vp(src_off), src_base, n, n_lanes, _vp(credits),
                                  credits.shape[0], epoch_len, quantum, tile_bytes, mode, _vp(st), _vp(table), _vp(hdr))
    if rc != 0:
        raise ValueError("fl_credit_schedule rejected its arguments")
    return table[:n], hdr[0], st[0]


def table_by_lane(table: np.ndarray, n_lanes: int, tiles_per_chunk: int) -> np.ndarray:
    table = np.ascontiguousarray(table)
    out = np.zeros(max(table.size, 1), dtype=DESC_DTYPE)
    if lib().fl_table_by_lane(_vp(table), table.size, n_lanes, tiles_per_chunk, _vp(out)) != 0:
        raise ValueError("fl_table_by_lane rejected its arguments")
    return out[: table.size]


def _window_ptrs(windows):
    arr = (C.c_void_p * MAX_LANES)()
    for l, w in enumerate(windows):
        arr[l] = w.ctypes.data
    return arr


def cpu_stripe(src: np.ndarray, table: np.ndarray, lane_caps):
    """Host memcpy striping: returns the list of lane windows (uint8 arrays of lane_caps bytes)."""
    windows = [np.zeros(max(int(c), 1), dtype=np.uint8) for c in lane_caps]
    ptrs = _window_ptrs(windows)
    table = np.ascontiguousarray(table)
    lib().fl_cpu_stripe(_vp(src), C.cast(ptrs, C.c_void_p), _vp(table), 0, table.size)
    return windows


def cpu_reassemble(nbytes: int, windows, table: np.ndarray) -> np.ndarray:
    dst = np.zeros(max(nbytes, 1), dtype=np.uint8)
    ptrs = _window_ptrs(windows)
    table = np.ascontiguousarray(table)
    lib().fl_cpu_reassemble(_vp(dst), C.cast(ptrs, C.c_void_p), _vp(table), 0, table.size)
    return dst[:nbytes]


def cpu_gather_pages(pool: np.ndarray, page_table: np.ndarray, page_bytes: int, ppc: int, table: np.ndarray, lane_caps):
    windows = [np.zeros(max(int(c), 1), dtype=np.uint8) for c in lane_caps]
    ptrs = _window_ptrs(windows)
    table = np.ascontiguousarray(table)
    page_table = np.ascontiguousarray(page_table, dtype=np.uint32)
    lib().fl_cpu_gather_pages(_vp(pool), _vp(page_table), page_bytes, ppc, C.cast(ptrs, C.c_void_p), _vp(table), table.size)
    return windows


def cpu_scatter_pages(pool_bytes: int, page_table: np.ndarray, page_bytes: int, ppc: int, windows, table: np.ndarray):
    pool = np.zeros(pool_bytes, dtype=np.uint8)
    ptrs = _window_ptrs(windows)
    table = np.ascontiguousarray(table)
    page_table = np.ascontiguousarray(page_table, dtype=np.uint32)
    lib().fl_cpu_scatter_pages(_vp(pool), _vp(page_table), page_bytes, ppc, C.cast(ptrs, C.c_void_p), _vp(table), table.size)
    return pool


def cpu_baseline(src: np.ndarray, table: np.ndarray, hdr: np.ndarray, n_lanes: int, threads: int, warm=3, iters=20):
    """Median and best seconds per stripe+reassemble on the host (memcpy)."""
    best = C.c_double()
    table = np.ascontiguousarray(table)
    hdr_arr = np.array([hdr], dtype=HDR_DTYPE)
    med = lib().fl_cpu_baseline_run(_vp(src), src.size, _vp(table), _vp(hdr_arr), table.size, n_lanes, threads, warm,
                                    iters, C.byref(best))
    if med < 0:
        raise RuntimeError(f"CPU baseline failed ({med})")
    return med, best.value
