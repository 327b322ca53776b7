"""ctypes binding of venom_amd/lib/libspatha.so (the C ABI of include/spatha.h).

The library is the only compute path of this package: if it is missing the
import of the binding fails loudly; there is no Python or CPU fallback.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
# SPATHA_LIBRARY names another build of the same library (e.g. the OUT_32B ablation build)
LIB_PATH = os.environ.get("SPATHA_LIBRARY") or os.path.join(_HERE, "lib", "libspatha.so")


class SpathaError(RuntimeError):
    def __init__(self, status, where):
        self.status = int(status)
        msg = _lib.spatha_status_string(int(status)).decode() if _lib is not None else "?"
        extra = ""
        if self.status == 4 and _lib is not None:
            extra = " (hipError %d)" % _lib.spatha_last_hip_error()
        super().__init__("%s: %s%s" % (where, msg, extra))


class Geometry(ctypes.Structure):
    _fields_ = [("rows", c_int32), ("cols", c_int32), ("n", c_int32), ("m", c_int32), ("v", c_int32),
                ("ksp", c_int32), ("n_values", c_int64), ("n_metadata", c_int64), ("n_columns", c_int64)]


# every symbol include/spatha.h declares, with its signature
SIGNATURES = {
    "spatha_status_string": (c_char_p, [c_int]),
    "spatha_last_hip_error": (c_int, []),
    "spatha_version": (c_char_p, []),
    "spatha_vnm_geometry_init": (c_int, [c_int, c_int, c_int, c_int, c_int, POINTER(Geometry)]),
    "spatha_vnm_random_pattern": (c_int, [c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "spatha_fill_rand_small_ints_f16": (c_int, [c_void_p, c_int64]),
    "spatha_benchmark_inputs_f16": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "spatha_vnm_encode_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int]),
    "spatha_vnm_encode_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int]),
    "spatha_vnm_decode_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int]),
    "spatha_vnm_decode_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int]),
    "spatha_vnm_select_columns_f32": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int]),
    "spatha_vnm_select_columns_f32_gpu": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "spatha_vnm_pack_meta_blob": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, POINTER(c_int64), POINTER(c_int64)]),
    "spatha_spmm_plan_create": (c_int, [c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(c_void_p)]),
    "spatha_spmm_plan_destroy": (c_int, [c_void_p]),
    "spatha_spmm_run": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "spatha_spmm_run_fused": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "spatha_spmm_run_noalloc": (c_int, [c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                        c_void_p, c_int, c_void_p]),
    "spatha_spmm_workspace_bytes": (ctypes.c_size_t, [c_void_p, c_int, c_int, c_int]),
    "spatha_spmm_workspace_init": (c_int, [c_void_p, ctypes.c_size_t, c_void_p]),
    "spatha_spmm_run_ws": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, ctypes.c_size_t, c_void_p]),
    "spatha_spmm_num_variants": (c_int, []),
    "spatha_spmm_kernel_name": (c_char_p, [c_void_p, c_int, c_int, c_int]),
    "spatha_spmm_time": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, POINTER(c_float)]),
    "spatha_spmm_tune": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, POINTER(c_int),
                                 POINTER(c_float), POINTER(c_float), POINTER(c_float)]),
    "spatha_dense_gemm_f16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "spatha_vnm_file_write": (c_int, [c_char_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "spatha_vnm_file_info": (c_int, [c_char_p, c_void_p, POINTER(c_int)]),
    "spatha_vnm_file_read": (c_int, [c_char_p, c_void_p, c_void_p, c_void_p]),
    "spatha_transpose_f16": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "spatha_add_layernorm_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_int, c_void_p, c_void_p]),
    "spatha_add_layernorm_f16_t": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p]),
}

_lib = None


def lib():
    """Loads libspatha.so (once).  Raises if the library has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "venom_amd: %s is missing; build it with `python -m venom_amd.build` "
                "(there is no fallback path)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status, where):
    if status != 0:
        raise SpathaError(status, where)
