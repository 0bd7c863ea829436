"""The C ABI: the library loads, exports every symbol include/rof.h declares, reports errors by code.
No compute call is made here (no GPU)."""
import ctypes as C
import os
import re

import pytest

from artifact_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


HEADERS = ("rof.h", "rof_bench.h")   # the library's interface and its benchmark / tuning interface


def _declared():
    names = set()
    for header in HEADERS:
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(rof_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_is_built_in_tree_and_loads():
    assert os.path.exists(_lib.LIB_PATH), "run `python -m artifact_amd.build`"
    assert _lib.lib().rof_version() >= 1


def test_every_declared_symbol_is_exported():
    L = _lib.lib()
    names = _declared()
    assert len(names) >= 25
    for name in names:
        assert hasattr(L, name), f"{name} is declared in include/ but not exported"
    assert set(_lib.SYMBOLS) == set(names)


def test_no_torch_types_in_signatures():
    for header in HEADERS:
        text = open(os.path.join(ROOT, "include", header)).read()
        assert "torch" not in text.lower() and "at::" not in text and "#include <hip" not in text


def test_benchmark_entry_points_are_not_in_the_product_header():
    text = open(os.path.join(ROOT, "include", "rof.h")).read()
    for name in ("rof_aggregate_timed", "rof_aggregate_launch_times", "rof_device_copy", "rof_device_read",
                 "rof_layout_set_tuning", "rof_layout_get_tuning"):
        assert name not in text


def test_error_codes_and_messages():
    L = _lib.lib()
    assert L.rof_strerror(0) == b"ok"
    for code, word in ((-1, b"argument"), (-2, b"range"), (-3, b"alloc"), (-4, b"HIP"), (-5, b"state"),
                       (-7, b"workspace")):
        assert word in L.rof_strerror(code)
    h = C.c_void_p()
    assert L.rof_split_part(None, 0, 3, C.byref(h)) == -1
    assert L.rof_plan_build(None, None, None, None, 0, 0, 3, 1, C.byref(h)) == -1
    assert L.rof_layout_from_v2(None, None, None, None, 0, 0, 3, None, C.byref(h)) == -1
    assert L.rof_aggregate(None, None, 0, 0, None, 0, 1, 1, None, 0, None) == -1
    assert L.rof_aggregate_noalloc(None, None, 0, 0, None, 0, 1, 1, None, None) == -1
    assert L.rof_layout_workspace_bytes(None, 4) == 0
    assert L.rof_layout_set_tuning(None, None) == -1 and L.rof_layout_get_tuning(None, None) == -1
    assert L.rof_layout_stats_n(None, None, 4) == -1
    assert L.rof_version() == 3
    ep = _lib.Epilogue(None, 1, 0, 0.5)
    assert L.rof_aggregate_epilogue(None, None, 0, 0, None, 0, 1, 1, C.byref(ep), None, 0, None) == -1
    assert L.rof_column_sums(None, 0, 4, 10, 4, None, None, 0, None) == -1          # no output
    out = (C.c_float * 4)()
    assert L.rof_column_sums(None, 0, 4, 10, 4, out, None, 0, None) == -1            # rows but no matrix
    assert L.rof_column_sums(out, 7, 4, 1, 4, out, out, 1 << 20, None) == -6         # unknown element type
    assert L.rof_column_sums(out, 0, 4, 1, 4, out, out, 16, None) == -7              # workspace too small
    assert L.rof_column_sums_workspace_bytes(1000, 47) == 2048 * 47 * 4 and L.rof_column_sums_workspace_bytes(0, 47) == 0
    assert L.rof_plan_hub_patterns(None, None, 0, 0, 16, 8, C.byref(h)) == -1
    assert L.rof_plan_dynamic_greedy(None, None, None, None, 0, 0, 3, C.byref(h)) == -1
    assert C.sizeof(_lib.Epilogue) == 32 and C.sizeof(_lib.LayoutOpts) == 48         # the structs of include/rof.h
    assert C.sizeof(_lib.LaunchTuning) == 32                                         # and of include/rof_bench.h
    with pytest.raises(_lib.RofError, match="invalid argument"):
        _lib.check(-1)


def test_operands_that_do_not_start_on_an_element_are_refused_before_any_launch():
    """x, out and the bias must start on a boundary of their element type; the check comes before the layout's state
    is looked at, so a layout that was never uploaded shows it (no HIP call is made)."""
    import numpy as np
    L = _lib.lib()
    ip = np.arange(0, 9, 2, dtype=np.int32)                       # 4 nodes x 2 neighbours
    ix = np.array([1, 2, 0, 3, 0, 3, 1, 2], dtype=np.int32)
    pn = np.arange(4, dtype=np.int32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    h = C.c_void_p()
    assert L.rof_layout_from_parts(p(ix), p(ip), p(pn), 4, 4, 2, None, C.byref(h)) == 0
    try:
        buf = (C.c_float * 64)()
        base = C.addressof(buf)
        agg = lambda x, dt, out: L.rof_aggregate(h, C.c_void_p(x), dt, 4, C.c_void_p(out), 4, 4, 0, None, 0, None)
        assert agg(base, 0, base + 64) == -5                      # aligned operands: only the upload is missing
        assert agg(base + 2, 0, base + 64) == -1                  # fp32 rows from a 2-byte boundary
        assert agg(base + 1, 1, base + 64) == -1                  # bf16 rows from an odd address
        assert agg(base + 2, 1, base + 64) == -5                  # bf16 rows from a 2-byte boundary are fine
        assert agg(base, 0, base + 66) == -1
        ep = _lib.Epilogue(C.c_void_p(base + 130), 0, 0, 0.0)
        assert L.rof_aggregate_epilogue(h, C.c_void_p(base), 0, 4, C.c_void_p(base + 64), 4, 4, 0, C.byref(ep), None, 0, None) == -1
    finally:
        L.rof_layout_free(h)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/librof.so")
    with pytest.raises(_lib.RofError, match="no fallback"):
        _lib.lib()
