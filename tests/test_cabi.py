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
    assert L.spatha_spmm_run(None, None, 8, None, None, 0, 0, None) == 1
    assert L.spatha_spmm_plan_destroy(None) == 0
    assert L.spatha_dense_gemm_f16(None, None, 8, 8, 8, None, None) == 1
    best, ms = ctypes.c_int(), ctypes.c_float()
    assert L.spatha_spmm_tune(None, None, 8, None, None, 0, 1, 1, None, None, None, None, None) == 1
    assert L.spatha_spmm_tune(None, None, 8, None, None, 0, 1, 1, None, ctypes.byref(best), ctypes.byref(ms), None, None) == 1


def test_unified_kernels_use_no_scratch_memory(tmp_path):
    """The unified dense-staged kernels load operands into registers asynchronously (inline assembly, no wait at the
    load); a register the compiler saves to scratch memory between such a load and its wait would hold a value that has
    not arrived.  Every instantiation shipped in the library must therefore have a private segment of zero bytes (the
    launcher checks the same at run time).  Read from the notes of the code objects embedded in libspatha.so."""
    import shutil
    import subprocess

    import pytest

    objdump, readelf = "/opt/rocm/llvm/bin/llvm-objdump", "/opt/rocm/llvm/bin/llvm-readelf"
    if not (os.path.exists(objdump) and os.path.exists(readelf)):
        pytest.skip("LLVM binary tools not present")
    lib = tmp_path / "libspatha.so"
    shutil.copy(_lib.LIB_PATH, lib)
    subprocess.check_call([objdump, "--offloading", str(lib)], cwd=tmp_path, stdout=subprocess.DEVNULL)
    found = {}
    for f in sorted(os.listdir(tmp_path)):
        if "amdgcn" not in f:
            continue
        notes = subprocess.check_output([readelf, "--notes", str(tmp_path / f)]).decode()
        name = None
        for line in notes.splitlines():
            line = line.strip()
            if line.startswith(".name:"):
                name = line.split(":", 1)[1].strip()
            elif line.startswith(".private_segment_fixed_size:") and name and ("spmm_du_kernel" in name or "spmm_up_kernel" in name):
                found[name] = int(line.split(":", 1)[1])
    assert len(found) >= 4, found                 # two output layouts x (m <= 8 in two phase groups, 8 < m <= 16)
    assert all(size == 0 for size in found.values()), found


def test_torch_extension_exposes_the_operator():
    """The PyTorch C++ extension is built in place and names the reference operator's fifteen arguments in order
    (end2end/spatha_mod/block_sparse/api/spatha.cu:41-65); calling it needs a GPU and is left to the GPU tests."""
    from venom_amd import spatha
    ext = spatha._extension()
    doc = ext.spmm.__doc__
    names = ["A_metadata", "A_indices", "A_values", "rhs_matrix", "bias", "A_num_rows", "A_num_cols", "B_num_cols",
             "vec_length", "n", "m", "nnz", "seed", "mbrow", "brow"]
    at = [doc.index(name + ":") for name in names]
    assert at == sorted(at)
    assert ext.plan_cache_size() == 0
    ext.clear_plan_cache()
