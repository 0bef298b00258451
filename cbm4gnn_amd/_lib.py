"""ctypes bindings of the two C-ABI libraries declared in ``include/cbm_hip.h``.

The libraries are loaded from ``cbm4gnn_amd/lib`` (built in-tree by ``cbm4gnn_amd.build``).
There is no fallback of any kind: a missing library raises ``CbmLibraryError`` and a non-zero
status from a call raises ``RuntimeError``.
"""
from __future__ import annotations

import ctypes as C
import os

from .build import HIP_LIB, HOST_LIB

CBM_OK = 0
CBM_PROP_SCALE_ROOTS = 1
CBM_SPMM_WORKSPACE_READY = 1
CBM_SPMM_RELU = 2
CBM_UPDATE_RELU = 2
CBM_UPDATE_WORKSPACE_READY = 4
CBM_SPMM_WORKSPACE_PRESCALED = 4
CBM_UPDATE_WORKSPACE_PRESCALED = 8
CBM_SPMM_SCHED_BATCHED = 8
CBM_UPDATE_SCHED_BATCHED = 16
CBM_ERR_NULL = 1
CBM_ERR_SHAPE = 3
CBM_ERR_SCRATCH = 7
CBM_STATIC_SCRATCH_FLOATS = 32 * 1024 * 1024
CBM_PATH_MAX_LEVELS = 16


class CbmLibraryError(RuntimeError):
    pass


class CbmFormat(C.Structure):
    """Mirror of ``struct cbm_format``."""
    _fields_ = [
        ("n", C.c_int32), ("n_levels", C.c_int32), ("is_symmetric", C.c_int32), ("reserved", C.c_int32), ("nnz", C.c_int64), ("nnz_a", C.c_int64),
        ("n_candidates", C.c_int64), ("msa_weight", C.c_int64),
        ("rowptr", C.POINTER(C.c_int32)), ("idx", C.POINTER(C.c_uint32)), ("parent", C.POINTER(C.c_int32)),
        ("order", C.POINTER(C.c_int32)), ("level_off", C.POINTER(C.c_int32)),
        ("mst_row", C.POINTER(C.c_int32)), ("mst_col", C.POINTER(C.c_int32)),
    ]


class CbmTiling(C.Structure):
    """Mirror of ``struct cbm_tiling`` (host arrays made by ``cbm_tile_rows``)."""
    _fields_ = [
        ("n", C.c_int32), ("tile_rows", C.c_int32), ("panel_rows", C.c_int32), ("n_panels", C.c_int32),
        ("n_blocks", C.c_int32), ("has_negative", C.c_int32),
        ("nnz_local", C.c_int64), ("nnz_local_padded", C.c_int64), ("nnz_remote", C.c_int64),
        ("panel_ptr", C.POINTER(C.c_int32)), ("blk_tile", C.POINTER(C.c_int32)), ("seg", C.POINTER(C.c_int32)),
        ("lidx", C.POINTER(C.c_uint16)), ("rowptr_r", C.POINTER(C.c_int32)), ("idx_r", C.POINTER(C.c_uint32)),
    ]


class CbmTilingDev(C.Structure):
    """Mirror of ``struct cbm_tiling_dev`` (the same arrays in device memory)."""
    _fields_ = [
        ("n_panels", C.c_int32), ("n_blocks", C.c_int32), ("tile_rows", C.c_int32), ("has_negative", C.c_int32),
        ("nnz_remote", C.c_int64),
        ("panel_ptr", C.c_void_p), ("blk_tile", C.c_void_p), ("seg", C.c_void_p), ("lidx", C.c_void_p),
        ("rowptr_r", C.c_void_p), ("idx_r", C.c_void_p), ("sched_r", C.c_void_p), ("row_scale", C.c_void_p),
        ("n_sched_r", C.c_int32), ("n_long", C.c_int32), ("n_pieces", C.c_int32), ("reserved", C.c_int32),
        ("long_rows", C.c_void_p),
    ]


class CbmWalkPlan(C.Structure):
    """Mirror of ``struct cbm_walk_plan`` (host arrays made by ``cbm_walk_plan_build``)."""
    _fields_ = [
        ("n", C.c_int32), ("cut", C.c_int32), ("n_entries", C.c_int32), ("n_bins", C.c_int32), ("n_slots", C.c_int32),
        ("reserved", C.c_int32), ("longest_bin", C.c_int64),
        ("entries", C.POINTER(C.c_int32)), ("bin_off", C.POINTER(C.c_int32)),
    ]


class CbmWalkDev(C.Structure):
    """Mirror of ``struct cbm_walk_dev`` (the same arrays in device memory)."""
    _fields_ = [
        ("cut", C.c_int32), ("n_entries", C.c_int32), ("n_bins", C.c_int32), ("n_slots", C.c_int32),
        ("entries", C.c_void_p), ("bin_off", C.c_void_p),
    ]


class CbmWalkStream(C.Structure):
    """Mirror of ``struct cbm_walk_stream`` (host arrays made by ``cbm_walk_stream_build``)."""
    _fields_ = [
        ("n", C.c_int32), ("n_bins", C.c_int32), ("n_slots", C.c_int32), ("n_elems", C.c_int32), ("heaviest_bin", C.c_int64),
        ("gidx", C.POINTER(C.c_uint32)), ("ginfo", C.POINTER(C.c_int32)), ("bin_goff", C.POINTER(C.c_int32)),
    ]


class CbmWalkStreamDev(C.Structure):
    """Mirror of ``struct cbm_walk_stream_dev`` (a multiply stream in device memory)."""
    _fields_ = [
        ("n", C.c_int32), ("n_bins", C.c_int32), ("n_slots", C.c_int32), ("n_elems", C.c_int32),
        ("gidx", C.c_void_p), ("ginfo", C.c_void_p), ("bin_goff", C.c_void_p),
    ]


CBM_WALK_LOAD_ONLY = 63
CBM_STREAM_LAST, CBM_STREAM_DUMMY, CBM_STREAM_COL_MASK = 0x40000000, 0x20000000, 0x1FFFFFFF
CBM_STREAM_ROW_COST = 5
CBM_WALK_MAX_SLOTS = 31

_P = C.c_void_p
_I32, _I64 = C.c_int32, C.c_int64

# name -> (restype, argtypes); the single list every symbol check iterates over
HOST_SYMBOLS = {
    "cbm_host_version": (C.c_char_p, []),
    "cbm_build_host": (C.c_int, [_P, _P, _I64, _I32, _I32, _I32, C.POINTER(CbmFormat)]),
    "cbm_format_free": (None, [C.POINTER(CbmFormat)]),
    "cbm_build_host_timings": (None, [C.POINTER(C.c_double)]),
    "cbm_schedule_rows": (C.c_int, [_P, _P, _P, _I32, _P]),
    "cbm_schedule_rows_batched": (C.c_int, [_P, _P, _P, _I32, _I32, _P]),
    "cbm_schedule_split_count": (C.c_int64, [_P, _I32, _I32, C.POINTER(C.c_int32)]),
    "cbm_schedule_rows_split": (C.c_int, [_P, _P, _P, _I32, _I32, _P, _P]),
    "cbm_schedule_blocks_count": (C.c_int64, [_P, _P, _I32, _I32, _I32, C.POINTER(C.c_int32)]),
    "cbm_schedule_rows_blocks": (C.c_int, [_P, _P, _P, _P, _I32, _I32, _I32, _P, _P]),
    "cbm_tile_rows": (C.c_int, [_P, _P, _I32, _I32, _I64, _I32, C.POINTER(CbmTiling)]),
    "cbm_tiling_free": (None, [C.POINTER(CbmTiling)]),
    "cbm_walk_plan_build": (C.c_int, [_P, _P, _P, _I32, _I32, _I32, _I32, C.POINTER(CbmWalkPlan)]),
    "cbm_walk_plan_free": (None, [C.POINTER(CbmWalkPlan)]),
    "cbm_walk_stream_build": (C.c_int, [_P, _P, _P, _P, _P, _I32, _I32, _I32, C.POINTER(CbmWalkStream)]),
    "cbm_walk_stream_free": (None, [C.POINTER(CbmWalkStream)]),
    "cbm_builder_create": (C.c_int, [_P, _P, _I64, _I32, _I32, C.POINTER(_P)]),
    "cbm_builder_arrays": (C.c_int, [_P, C.POINTER(_P), C.POINTER(_P), C.POINTER(_P), C.POINTER(_P), C.POINTER(_P),
                                     C.POINTER(_P), C.POINTER(_I64)]),
    "cbm_builder_finish": (C.c_int, [_P, _I32, _P, _I64, C.POINTER(CbmFormat)]),
    "cbm_builder_set_max_levels": (C.c_int, [_P, _I32]),
    "cbm_builder_free": (None, [_P]),
}
HIP_SYMBOLS = {
    "cbm_version": (C.c_char_p, []),
    "cbm_status_string": (C.c_char_p, [C.c_int]),
    "cbm_set_spmm_kernel": (C.c_int, [C.c_int]),
    "cbm_set_spmm_occupancy": (C.c_int, [C.c_int]),
    "cbm_spmm_summation_groups": (C.c_int, [_I32, _I64, _I64, _P, _P, _I32]),
    "cbm_spmm_tail_columns": (C.c_int, [_I32, _I64, _I64, _P, _P, _I32]),
    "cbm_set_tiled_fused": (C.c_int, [C.c_int]),
    "cbm_relayout_floats": (C.c_int64, [_I32, _I32]),
    "cbm_spmm_workspace_floats": (C.c_int64, [_I32, _I32, _I64, _I64, _P, _P]),
    "cbm_expand_coef_f32": (C.c_int, [_P, _P, _P, _I64, _P]),
    "cbm_spmm_f32": (C.c_int, [_P, _P, _I64, _P, _P, _P, _P, _P, _P, _P, _I32, _I32, _I32, _I64, _I64, _P]),
    "cbm_relayout_slabs_f32": (C.c_int, [_P, _P, _I32, _I32, _I64, _P]),
    "cbm_relayout_slabs_masked_f32": (C.c_int, [_P, _P, _P, _P, _I32, _I32, _I64, _I64, _P]),
    "cbm_relayout_slabs_scaled_f32": (C.c_int, [_P, _P, _P, _I32, _I32, _I64, _P]),
    "cbm_propagate_f32": (C.c_int, [_P, _P, _P, _P, _I32, _P, _P, _I32, _I32, _I64, _I32, _P]),
    "cbm_propagate_subtrees_f32": (C.c_int, [C.POINTER(CbmWalkDev), _P, _P, _P, _P, _I32, _P, _P, _I32, _I32, _I64, _I32, _P]),
    "cbm_spmm_update_subtrees_f32": (C.c_int, [C.POINTER(CbmWalkStreamDev), _P, _P, _P, _I32, _I32, _I64, _I64, _I32, _P]),
    "cbm_spmm_update_f32": (C.c_int, [_P, _P, _I64, _P, _P, _P, _P, _P, _P, _P, _I32, _P, _P, _P, _I32, _I32, _I64, _I64, _I32, _P]),
    "cbm_spmm_update_paths_f32": (C.c_int, [_P, _P, _I64, _P, _P, _P, _P, _P, _P, _P, _I32, _P, _P, _P, _P, _I32, _I32, _I64, _I64, _I32, _P]),
    "cbm_spmm_update_single_f32": (C.c_int, [_P, _P, _P, _P, _P, _I32, _P, _P, _I32, _I32, _I64, _I64, _I32, _P]),
    "cbm_spmm_update_paths_scratch_floats": (C.c_int64, [_I32, _I32, _I32]),
    "cbm_spmm_update_static_f32": (C.c_int, [_P, _P, _I64, _P, _P, _P, _P, _P, _P, _P, _I32, _P, _P, _I32, _I32, _I64, _I64, _I32, _P]),
    "cbm_spmm_tiled_workspace_floats": (C.c_int64, [C.POINTER(CbmTilingDev), _I32, _I32]),
    "cbm_spmm_tiled_f32": (C.c_int, [C.POINTER(CbmTilingDev), _P, _P, _P, _P, _I32, _I32, _I32, _I64, _I64, _P]),
    "cbm_spmm_update_tiled_f32": (C.c_int, [C.POINTER(CbmTilingDev), _P, _P, _P, _P, _P, _I32, _P, _P, _P, _I32, _I32, _I64,
                                            _I64, _I32, _P]),
    "csr_spmm_f32": (C.c_int, [_P, _P, _I64, _P, _P, _P, _P, _P, _I32, _I32, _I32, _I64, _I64, _P]),
    "cbm_row_intersections_groups": (C.c_int, []),
    "cbm_row_intersections": (C.c_int, [_P, _P, _P, _P, _P, _P, _I32, _I32, _I32, _P, _P, _I64, _P, _P]),
}

_host = None
_hip = None


def _load(path: str, symbols: dict, what: str):
    if not os.path.exists(path):
        raise CbmLibraryError(
            f"{what} library not found at {path}; build it with `python -m cbm4gnn_amd.build` "
            "(there is no CPU fallback)")
    try:
        lib = C.CDLL(path)
    except OSError as e:                                   # e.g. libamdhip64 missing
        raise CbmLibraryError(f"cannot load {path}: {e}") from e
    for name, (res, args) in symbols.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise CbmLibraryError(f"{path} does not export {name}") from e
        fn.restype = res
        fn.argtypes = args
    return lib


def host_lib():
    global _host
    if _host is None:
        _host = _load(HOST_LIB, HOST_SYMBOLS, "host builder")
    return _host


def hip_lib():
    global _hip
    if _hip is None:
        _hip = _load(HIP_LIB, HIP_SYMBOLS, "HIP kernel")
    return _hip


def check(status: int, where: str):
    if status != CBM_OK:
        msg = hip_lib().cbm_status_string(status).decode() if _hip is not None else f"status {status}"
        exc = ValueError if status in (1, 3) else RuntimeError
        raise exc(f"{where}: {msg} (status {status})")
