"""ctypes binding of librof.so (the C ABI declared in include/rof.h).

There is no CPU fallback: if the library has not been built, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librof.so")
_lib = None

# every symbol include/rof.h declares (checked by the CPU test-suite against the header text)
SYMBOLS = (
    "rof_strerror", "rof_last_device_error", "rof_version", "rof_bag_get", "rof_bag_free", "rof_split_part",
    "rof_part_intersect_count", "rof_part_intersect_lists", "rof_greedy_max_reuse", "rof_reorganize",
    "rof_transpose_csr", "rof_plan_build", "rof_layout_from_v2", "rof_layout_from_v1", "rof_layout_from_parts",
    "rof_layout_export", "rof_layout_stats", "rof_layout_upload", "rof_layout_set_degrees",
    "rof_plan_hub_patterns", "rof_plan_dynamic_greedy", "rof_column_sums", "rof_column_sums_workspace_bytes", "rof_layout_workspace_bytes", "rof_layout_free", "rof_aggregate", "rof_aggregate_epilogue", "rof_aggregate_noalloc", "rof_aggregate_timed", "rof_aggregate_launch_times",
    "rof_device_copy", "rof_device_read", "rof_device_gather", "rof_layout_set_tuning", "rof_layout_get_tuning", "rof_layout_stats_n", "rof_layout_calibrate",
)


class RofError(RuntimeError):
    pass


class LayoutOpts(C.Structure):
    _fields_ = [("min_consumers", C.c_int32), ("disable_reuse", C.c_int32), ("hub_split", C.c_int32),
                ("segment", C.c_int32), ("lanes_per_row", C.c_int32), ("entry_order", C.c_int32),
                ("tile_rows", C.c_int32), ("elem_bytes", C.c_int32), ("local_groups", C.c_int32),
                ("share_scope", C.c_int32), ("row_bytes", C.c_int32), ("reserved", C.c_int32 * 1)]


class LaunchTuning(C.Structure):
    _fields_ = [("xcd_run_partial", C.c_int32), ("xcd_run_dst", C.c_int32), ("wave_cap", C.c_int32),
                ("lds_pad", C.c_int32), ("deep", C.c_int32), ("reserved", C.c_int32 * 3)]


class Epilogue(C.Structure):
    _fields_ = [("bias", C.c_void_p), ("relu", C.c_int32), ("out_dtype", C.c_int32), ("self_weight", C.c_float),
                ("pad_columns", C.c_int32), ("reserved", C.c_int32 * 2)]


def lib():
    """Load librof.so once.  Raises if it is missing: build it with `python -m artifact_amd.build`."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RofError(f"{LIB_PATH} is not built (run `python -m artifact_amd.build`); there is no fallback path")
    L = C.CDLL(LIB_PATH)
    vp, u32, u64, i32, i64, ci = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int32, C.c_int64, C.c_int
    pp = C.POINTER(C.c_void_p)
    L.rof_strerror.restype = C.c_char_p
    L.rof_strerror.argtypes = [ci]
    L.rof_last_device_error.restype = C.c_char_p
    L.rof_version.restype = ci
    L.rof_bag_get.restype = i64
    L.rof_bag_get.argtypes = [vp, C.c_char_p, pp]
    L.rof_bag_free.argtypes = [vp]
    L.rof_split_part.argtypes = [vp, u32, ci, pp]
    L.rof_part_intersect_count.argtypes = [vp, u64, vp, u64, vp, vp, u32, ci, ci, pp]
    L.rof_part_intersect_lists.argtypes = [vp, u64, vp, u64, vp, vp, u32, ci, ci, vp, u64, pp]
    L.rof_greedy_max_reuse.argtypes = [vp, u64, vp, vp, u64, pp]
    L.rof_reorganize.argtypes = [vp, u64, vp, u64, vp, u64, vp, vp, vp, u32, vp, ci, ci, pp]
    L.rof_transpose_csr.argtypes = [vp, vp, u32, u64, pp]
    L.rof_plan_build.argtypes = [vp, vp, vp, vp, u32, u64, ci, ci, pp]
    L.rof_plan_hub_patterns.argtypes = [vp, vp, u32, u64, u32, ci, pp]
    L.rof_plan_dynamic_greedy.argtypes = [vp, vp, vp, vp, u32, u64, ci, pp]
    L.rof_layout_from_v2.argtypes = [vp, vp, vp, vp, i64, i32, ci, vp, pp]
    L.rof_layout_from_v1.argtypes = [vp, vp, vp, i64, vp, vp, vp, i64, i32, ci, vp, pp]
    L.rof_layout_from_parts.argtypes = [vp, vp, vp, i64, i32, ci, vp, pp]
    L.rof_layout_export.argtypes = [vp, pp]
    L.rof_layout_stats.argtypes = [vp, vp]
    L.rof_layout_upload.argtypes = [vp, vp]
    L.rof_layout_set_degrees.argtypes = [vp, vp, vp]
    L.rof_layout_workspace_bytes.restype = C.c_size_t
    L.rof_layout_workspace_bytes.argtypes = [vp, ci]
    L.rof_layout_free.argtypes = [vp]
    L.rof_aggregate.argtypes = [vp, vp, ci, i64, vp, i64, ci, ci, vp, C.c_size_t, vp]
    L.rof_aggregate_epilogue.argtypes = [vp, vp, ci, i64, vp, i64, ci, ci, C.POINTER(Epilogue), vp, C.c_size_t, vp]
    L.rof_aggregate_noalloc.argtypes = [vp, vp, ci, i64, vp, i64, ci, ci, C.POINTER(Epilogue), vp]
    L.rof_aggregate_timed.argtypes = [vp, vp, ci, i64, vp, i64, ci, ci, C.POINTER(Epilogue), vp, C.c_size_t, vp, ci,
                                      C.POINTER(C.c_float)]
    L.rof_layout_set_tuning.argtypes = [vp, C.POINTER(LaunchTuning)]
    L.rof_layout_get_tuning.argtypes = [vp, C.POINTER(LaunchTuning)]
    L.rof_layout_stats_n.argtypes = [vp, vp, ci]
    L.rof_layout_calibrate.argtypes = [vp, vp, ci, i64, vp, i64, ci, ci, C.POINTER(Epilogue), vp, C.c_size_t, vp, ci, ci,
                                       C.POINTER(LaunchTuning)]
    L.rof_device_read.argtypes = [vp, C.c_size_t, ci, vp, vp]
    L.rof_device_gather.argtypes = [vp, u32, ci, ci, vp, vp, C.POINTER(C.c_uint64)]
    L.rof_column_sums_workspace_bytes.argtypes = [i64, ci]
    L.rof_column_sums_workspace_bytes.restype = C.c_size_t
    L.rof_column_sums.argtypes = [vp, ci, i64, i64, ci, vp, vp, C.c_size_t, vp]
    L.rof_device_copy.argtypes = [vp, vp, C.c_size_t, vp]
    L.rof_aggregate_launch_times.argtypes = [vp, vp, ci, i64, vp, i64, ci, ci, C.POINTER(Epilogue), vp, C.c_size_t, vp, ci,
                                             C.POINTER(C.c_float * 2)]
    _lib = L
    return L


def check(status):
    if status != 0:
        L = lib()
        msg = L.rof_strerror(status).decode()
        if status == -4:
            msg += ": " + L.rof_last_device_error().decode()
        raise RofError(f"librof: {msg} (status {status})")


def u32(a):
    """numpy uint32, C-contiguous; int32 input is reinterpreted like pybind's forcecast does upstream."""
    a = np.asarray(a)
    if a.dtype != np.uint32:
        a = a.astype(np.uint32)
    return np.ascontiguousarray(a).ravel()


def i32(a):
    a = np.asarray(a)
    if a.dtype != np.int32:
        a = a.astype(np.int32)
    return np.ascontiguousarray(a).ravel()


def ptr(a):
    return a.ctypes.data if a is not None and a.size else None


def bag_take(handle, names, dtype=np.uint32, free=True):
    """Copy named arrays out of a bag into numpy arrays and release the bag."""
    L = lib()
    out = {}
    try:
        for name in names:
            p = C.c_void_p()
            n = L.rof_bag_get(handle, name.encode(), C.byref(p))
            if n < 0:
                raise RofError(f"librof: result has no array '{name}'")
            if n == 0:
                out[name] = np.empty(0, dtype=dtype)
            else:
                buf = (C.c_uint32 * n).from_address(p.value)
                out[name] = np.frombuffer(buf, dtype=np.uint32).copy().view(dtype)
    finally:
        if free:
            L.rof_bag_free(handle)
    return out
