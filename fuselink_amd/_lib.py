"""ctypes binding of libnccl-net-fuselink.so.  There is no fallback: if the library is missing or a
symbol is absent, importing a wrapper that needs it raises."""
from __future__ import annotations

import ctypes as C
import os

from .build import lib_path

MAX_LANES = 16


class ChunkDesc(C.Structure):
    _fields_ = [("src_off", C.c_uint64), ("win_off", C.c_uint64), ("len", C.c_uint32), ("lane", C.c_uint32),
                ("tile_base", C.c_uint32), ("epoch", C.c_uint32)]


class SchedState(C.Structure):
    _fields_ = [("epoch_bytes", C.c_uint64), ("chunk_index", C.c_uint64), ("lane_off", C.c_uint64 * MAX_LANES)]


class SchedHdr(C.Structure):
    _fields_ = [("total_bytes", C.c_uint64), ("total_tiles", C.c_uint32), ("n_chunks", C.c_uint32),
                ("flags", C.c_uint32), ("uniform_tiles", C.c_uint32), ("lane_bytes", C.c_uint64 * MAX_LANES),
                ("lane_chunks", C.c_uint32 * MAX_LANES)]


class SchedParams(C.Structure):
    _fields_ = [("d_sizes", C.c_void_p), ("total_bytes", C.c_uint64), ("chunk_bytes", C.c_uint32),
                ("d_src_off", C.c_void_p), ("src_base", C.c_uint64), ("n_chunks", C.c_uint32),
                ("n_lanes", C.c_uint32), ("d_credits", C.c_void_p), ("n_rows", C.c_uint32),
                ("epoch_len", C.c_uint32), ("quantum", C.c_uint64), ("tile_bytes", C.c_uint32),
                ("mode", C.c_uint32), ("d_state", C.c_void_p), ("d_table", C.c_void_p), ("d_hdr", C.c_void_p),
                ("inline_credits", C.c_uint32 * MAX_LANES), ("d_table_by_lane", C.c_void_p),
                ("d_tiles", C.c_void_p), ("tiles_cap", C.c_uint32), ("pad_", C.c_uint32),
                ("d_workspace", C.c_void_p), ("workspace_bytes", C.c_uint64), ("wave_chunks", C.c_uint32), ("pad2_", C.c_uint32)]


class UniformParams(C.Structure):
    _fields_ = [("total_bytes", C.c_uint64), ("src_base", C.c_uint64), ("epoch_bytes", C.c_uint64),
                ("chunk_bytes", C.c_uint32), ("n_lanes", C.c_uint32), ("tile_bytes", C.c_uint32), ("pad", C.c_uint32),
                ("credits", C.c_uint32 * MAX_LANES), ("d_done_word", C.c_void_p), ("d_done_count", C.c_void_p),
                ("done_value", C.c_uint32), ("start_value", C.c_uint32), ("done_event", C.c_void_p), ("d_start_word", C.c_void_p)]


BATCH_MAX = 32
SEG_MAX = 8


class BatchSegment(C.Structure):
    _fields_ = [("epoch_bytes", C.c_uint64), ("n_req", C.c_uint32), ("pad", C.c_uint32), ("credits", C.c_uint32 * MAX_LANES)]


class BatchParams(C.Structure):
    _fields_ = [("u", UniformParams), ("n_req", C.c_uint32), ("n_seg", C.c_uint32), ("d_src", C.c_void_p * BATCH_MAX),
                ("d_dst", C.c_void_p * BATCH_MAX), ("bytes", C.c_uint64 * BATCH_MAX), ("seg", BatchSegment * SEG_MAX)]


class Windows(C.Structure):
    _fields_ = [("base", C.c_void_p * MAX_LANES), ("cap", C.c_uint64 * MAX_LANES), ("n_lanes", C.c_uint32),
                ("pad", C.c_uint32)]


# name -> (restype, argtypes); every symbol declared in include/fuselink_hip.h
SIGNATURES = {
    "flh_init": (C.c_int, [C.c_int]),
    "flh_last_error": (C.c_char_p, []),
    "flh_constant": (C.c_int64, [C.c_int]),
    "flh_schedule_workspace_bytes": (C.c_uint64, [C.c_uint32]),
    "flh_schedule": (C.c_int, [C.POINTER(SchedParams), C.c_void_p]),
    "flh_schedule_static": (C.c_int, [C.POINTER(SchedParams), C.c_void_p]),
    "flh_stripe": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(Windows), C.c_void_p, C.c_void_p, C.POINTER(SchedHdr),
                             C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]),
    "flh_reassemble": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(Windows), C.c_void_p, C.c_void_p,
                                 C.POINTER(SchedHdr), C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]),
    "flh_stripe_tiles": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(Windows), C.c_void_p, C.c_uint32, C.c_void_p, C.POINTER(SchedHdr),
                                   C.c_void_p, C.c_void_p]),
    "flh_reassemble_tiles": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(Windows), C.c_void_p, C.c_uint32, C.c_void_p, C.POINTER(SchedHdr),
                                       C.c_void_p, C.c_void_p]),
    "flh_stripe_uniform": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(Windows), C.POINTER(UniformParams), C.c_void_p,
                                     C.c_void_p, C.c_void_p, C.c_void_p]),
    "flh_reassemble_uniform": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(Windows), C.POINTER(UniformParams), C.c_void_p,
                                         C.c_void_p]),
    "flh_stripe_uniform_carry": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(Windows), C.POINTER(Windows), C.POINTER(UniformParams), C.c_void_p,
                                           C.c_void_p, C.c_void_p, C.c_void_p]),
    "flh_stripe_batch_carry": (C.c_int, [C.POINTER(BatchParams), C.POINTER(Windows), C.POINTER(Windows), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "flh_stage_deliver_batch": (C.c_int, [C.POINTER(BatchParams), C.POINTER(Windows), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "flh_stage_deliver_uniform": (C.c_int, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64, C.POINTER(Windows), C.POINTER(UniformParams), C.c_void_p,
                                            C.c_void_p, C.c_void_p, C.c_void_p]),
    "flh_engine_submit_wire": (C.c_int, [C.c_void_p, C.c_uint32, C.POINTER(BatchParams), C.POINTER(Windows), C.POINTER(Windows), C.c_void_p, C.c_void_p,
                                         C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "flh_engine_set_resident": (C.c_int, [C.c_void_p, C.c_uint32]),
    "flh_engine_trace": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint32, C.c_void_p]),
    "flh_engine_needs_start": (C.c_int, [C.c_void_p]),
    "flh_engine_poke": (C.c_int, [C.c_void_p]),
    "flh_window_export_dmabuf": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64, C.POINTER(C.c_int)]),
    "flh_stripe_batch": (C.c_int, [C.POINTER(BatchParams), C.POINTER(Windows), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "flh_reassemble_batch": (C.c_int, [C.POINTER(BatchParams), C.POINTER(Windows), C.c_void_p, C.c_void_p]),
    "flh_engine_create": (C.c_int, [C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.POINTER(C.c_void_p)]),
    "flh_engine_submit": (C.c_int, [C.c_void_p, C.POINTER(BatchParams), C.POINTER(Windows), C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_uint64),
                                    C.POINTER(C.c_uint64)]),
    "flh_engine_completed": (C.c_uint64, [C.c_void_p]),
    "flh_engine_error": (C.c_int, [C.c_void_p]),
    "flh_engine_launches": (C.c_uint64, [C.c_void_p]),
    "flh_engine_destroy": (C.c_int, [C.c_void_p]),
    "flh_batch_layout": (C.c_int, [C.POINTER(BatchParams), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "flh_gather_pages": (C.c_int, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint32, C.c_uint32, C.POINTER(Windows),
                                   C.c_void_p, C.c_uint32, C.c_int, C.c_void_p, C.c_void_p]),
    "flh_scatter_pages": (C.c_int, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint32, C.c_uint32, C.POINTER(Windows),
                                    C.c_void_p, C.c_uint32, C.c_int, C.c_void_p, C.c_void_p]),
    "flh_gather_pages_uniform": (C.c_int, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint32, C.POINTER(Windows),
                                           C.POINTER(UniformParams), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "flh_scatter_pages_uniform": (C.c_int, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint32, C.POINTER(Windows),
                                            C.POINTER(UniformParams), C.c_void_p, C.c_void_p]),
    "flh_copy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p]),
    "flh_copy_runs": (C.c_int, [C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_uint64), C.c_uint32, C.c_void_p]),
    "flh_qp_split": (C.c_int, [C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "flh_pool_create": (C.c_int, [C.c_int, C.c_uint32, C.POINTER(C.c_void_p)]),
    "flh_pool_destroy": (C.c_int, [C.c_void_p]),
    "flh_pool_free_units": (C.c_int, [C.c_void_p]),
    "flh_pool_slot_of": (C.c_int, [C.c_void_p, C.c_void_p]),
    "flh_pool_granularity": (C.c_uint64, [C.c_void_p]),
    "flh_window_create": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(C.c_void_p)]),
    "flh_window_bind": (C.c_int, [C.c_void_p, C.c_uint64]),
    "flh_window_trim": (C.c_int, [C.c_void_p, C.c_uint64]),
    "flh_window_destroy": (C.c_int, [C.c_void_p]),
    "flh_window_base": (C.c_void_p, [C.c_void_p]),
    "flh_window_bound_bytes": (C.c_uint64, [C.c_void_p]),
    "flh_window_slots": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.c_int]),
    "flh_region_acquire": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint32, C.c_uint64,
                                     C.POINTER(C.c_void_p)]),
    "flh_region_release": (C.c_int, [C.c_void_p]),
    "flh_region_refs": (C.c_int, [C.c_void_p]),
    "flh_region_windows": (C.c_int, [C.c_void_p, C.POINTER(Windows)]),
    "flh_region_translate": (C.c_void_p, [C.c_void_p, C.c_uint32, C.c_void_p]),
    "flh_tune": (C.c_int, [C.c_char_p, C.c_int64]),
    "flh_prof_begin": (C.c_int, [C.c_int]),
    "flh_prof_end": (C.c_int, [C.POINTER(C.c_double), C.POINTER(C.c_int), C.c_int]),
}

_lib = None


def load() -> C.CDLL:
    """Loads the in-tree library (built beforehand by ``python -m fuselink_amd.build``)."""
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("FUSELINK_LIB", lib_path())
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `python -m fuselink_amd.build` "
                          "(there is no CPU or PyTorch fallback for this path)")
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class FuseLinkError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"fuselink error {code}: {msg}")
        self.code = code


def check(rc: int) -> int:
    if rc < 0:
        raise FuseLinkError(rc, load().flh_last_error().decode(errors="replace"))
    return rc
