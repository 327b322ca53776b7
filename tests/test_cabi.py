"""The C-ABI library loads and exports every symbol include/spatha.h declares."""
import ctypes
import os
import re

from venom_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "spatha.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(spatha_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    names = _declared_symbols()
    assert len(names) >= 18
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(raw, name), name
    assert set(names) == set(_lib.SIGNATURES), set(names) ^ set(_lib.SIGNATURES)


def test_status_strings_and_version():
    L = _lib.lib()
    assert L.spatha_version().decode().count(".") == 2
    seen = {L.spatha_status_string(i).decode() for i in range(7)}
    assert len(seen) == 7 and "ok" in seen


def test_spmm_entry_points_reject_bad_arguments_without_a_gpu():
    L = _lib.lib()
    handle = ctypes.c_void_p()
    # null arrays
    assert L.spatha_spmm_plan_create(128, 128, 2, 8, 64, None, None, None, None, ctypes.byref(handle)) == 1
    # shape errors come before any device work
    assert L.spatha_spmm_plan_create(100, 128, 2, 8, 64, 1, 1, 1, None, ctypes.byref(handle)) == 2
    assert L.spatha_spmm_plan_create(96, 128, 2, 8, 32, 16, 16, 16, None, ctypes.byref(handle)) == 3   # rows % 64: no kernel
    assert L.spatha_spmm_run(None, None, 8, None, None, 0, 0, None) == 1
    assert L.spatha_spmm_plan_destroy(None) == 0
    assert L.spatha_dense_gemm_f16(None, None, 8, 8, 8, None, None) == 1
