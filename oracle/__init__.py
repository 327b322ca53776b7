"""numpy front-end of the CPU oracle (oracle/vnm_oracle.cpp).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's cpu_baseline leg.  Nothing under venom_amd/ imports it.
"""
import ctypes
import os

import numpy as np

from . import build as _build

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "libvnm_oracle.so")
        if not os.path.exists(path):
            _build.build(force=True)
        L = ctypes.CDLL(path)
        L.vo_rand.restype = ctypes.c_int
        L.vo_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def sizes(rows, cols, n, m, v):
    out = np.zeros(4, dtype=np.int64)
    lib().vo_sizes(rows, cols, n, m, v, _p(out))
    return dict(ksp=int(out[0]), n_values=int(out[1]), n_metadata=int(out[2]), n_columns=int(out[3]))


def half_to_float(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().vo_half_to_float(_p(h), _p(out), ctypes.c_long(h.size))
    return out


def float_to_half(f):
    f = _c(f, np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().vo_float_to_half(_p(f), _p(out), ctypes.c_long(f.size))
    return out


def add_half(a, b):
    a = _c(a, np.uint16)
    b = _c(b, np.uint16)
    out = np.empty(a.shape, np.uint16)
    lib().vo_add_half(_p(a), _p(b), _p(out), ctypes.c_long(a.size))
    return out


def srand(seed=1):
    lib().vo_srand(ctypes.c_uint(seed))


def random_mask(rows, cols, n, m, v, mbrow=32):
    s = sizes(rows, cols, n, m, v)
    meta = np.zeros(s["n_metadata"], np.uint32)
    columns = np.zeros(s["n_columns"], np.uint32)
    lib().vo_random_mask(rows, cols, n, m, v, mbrow, _p(meta), _p(columns))
    return meta, columns


def shuffle(a):
    """One draw of the generator's shuffle on the process-wide rand() stream (a copy of `a`, shuffled)."""
    a = np.array(a, dtype=np.uint32)
    lib().vo_shuffle(_p(a), int(a.size))
    return a


def fill_rand_ints(count):
    out = np.empty(count, np.float32)
    lib().vo_fill_rand_ints(_p(out), ctypes.c_long(count))
    return out


def encode(dense, columns, n, m, v, mask=None):
    """dense: float32 or float16 (rows, cols).  Returns (values, metadata)."""
    rows, cols = dense.shape
    s = sizes(rows, cols, n, m, v)
    columns = _c(columns, np.uint32).reshape(-1)
    assert columns.size == s["n_columns"], (columns.size, s)
    meta = np.zeros(s["n_metadata"], np.uint32)
    mk = None if mask is None else _c(mask, np.int32)
    if dense.dtype == np.float16:
        d = np.ascontiguousarray(dense).view(np.uint16)
        values = np.zeros(s["n_values"], np.uint16)
        lib().vo_encode_f16(_p(d), _p(mk), _p(columns), rows, cols, n, m, v, _p(values), _p(meta))
        return values.view(np.float16), meta
    d = _c(dense, np.float32)
    values = np.zeros(s["n_values"], np.float32)
    lib().vo_encode_f32(_p(d), _p(mk), _p(columns), rows, cols, n, m, v, _p(values), _p(meta))
    return values, meta


def decode(values, meta, columns, rows, cols, n, m, v):
    columns = _c(columns, np.uint32).reshape(-1)
    meta = _c(meta, np.uint32)
    if values.dtype == np.float16:
        vals = np.ascontiguousarray(values).view(np.uint16)
        dense = np.zeros((rows, cols), np.uint16)
        lib().vo_decode_f16(_p(vals), _p(meta), _p(columns), rows, cols, n, m, v, _p(dense))
        return dense.view(np.float16)
    vals = _c(values, np.float32)
    dense = np.zeros((rows, cols), np.float32)
    lib().vo_decode_f32(_p(vals), _p(meta), _p(columns), rows, cols, n, m, v, _p(dense))
    return dense


def select_columns(dense_abs, n, m, v, want_sparse=False):
    d = _c(dense_abs, np.float32)
    rows, cols = d.shape
    s = sizes(rows, cols, n, m, v)
    masks = np.zeros((rows, cols), np.int32)
    columns = np.zeros(s["n_columns"], np.int32)
    sp = d.copy() if want_sparse else None
    lib().vo_select_columns(_p(d), _p(sp), rows, cols, n, m, v, _p(masks), _p(columns))
    return (masks, columns, sp) if want_sparse else (masks, columns)


def spmm(values, meta, columns, rows, cols, n, m, v, B, bias=None, transposed_out=False, threads=0):
    """fp16 SpMM on the compressed form; returns fp16 C (rows, N) or (N, rows)."""
    vals = np.ascontiguousarray(values, dtype=np.float16).view(np.uint16)
    meta = _c(meta, np.uint32)
    columns = _c(columns, np.uint32).reshape(-1)
    Bh = np.ascontiguousarray(B, dtype=np.float16)
    assert Bh.shape[0] == cols
    N = Bh.shape[1]
    bh = None if bias is None else np.ascontiguousarray(bias, dtype=np.float16).view(np.uint16)
    C = np.zeros((N, rows) if transposed_out else (rows, N), np.uint16)
    lib().vo_spmm_f16(_p(vals), _p(meta), _p(columns), rows, cols, n, m, v, _p(Bh.view(np.uint16)), N, _p(bh),
                      1 if transposed_out else 0, _p(C), threads)
    return C.view(np.float16)


def dense_gemm(A, B, threads=0):
    Ah = np.ascontiguousarray(A, dtype=np.float16)
    Bh = np.ascontiguousarray(B, dtype=np.float16)
    rows, cols = Ah.shape
    N = Bh.shape[1]
    C = np.zeros((rows, N), np.uint16)
    lib().vo_dense_gemm_f16(_p(Ah.view(np.uint16)), _p(Bh.view(np.uint16)), rows, cols, N, _p(C), threads)
    return C.view(np.float16)


def check_results(a, b):
    a = np.ascontiguousarray(a, dtype=np.float16).view(np.uint16)
    b = np.ascontiguousarray(b, dtype=np.float16).view(np.uint16)
    return int(lib().vo_check_results(_p(a), _p(b), ctypes.c_long(a.size)))


def num_threads():
    return int(lib().vo_num_threads())
