"""Host side of the V:N:M format for Python callers: numpy in, numpy out, all
work done by libspatha.so (OpenMP C++).  Mirrors the reference's host helpers
(end2end/grouped_nmv_tensor.py and src/format/format_sr_nm.cpp)."""
import ctypes

import numpy as np

from . import _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def geometry(rows, cols, n, m, v):
    g = _lib.Geometry()
    _lib.check(_lib.lib().spatha_vnm_geometry_init(rows, cols, n, m, v, ctypes.byref(g)), "spatha_vnm_geometry_init")
    return g


def encode(dense, columns, n, m, v, mask=None, threads=0):
    """dense (rows, cols) float32 or float16 -> (values, metadata uint32)."""
    dense = np.ascontiguousarray(dense)
    rows, cols = dense.shape
    g = geometry(rows, cols, n, m, v)
    columns = np.ascontiguousarray(columns, dtype=np.uint32).reshape(-1)
    if columns.size != g.n_columns:
        raise ValueError("columns has %d entries, the format needs %d" % (columns.size, g.n_columns))
    mk = None if mask is None else np.ascontiguousarray(mask, dtype=np.int32)
    if mk is not None and mk.shape != dense.shape:
        raise ValueError("mask shape differs from dense shape")
    meta = np.zeros(g.n_metadata, np.uint32)
    L = _lib.lib()
    if dense.dtype == np.float16:
        values = np.zeros(g.n_values, np.float16)
        st = L.spatha_vnm_encode_f16(_p(dense), _p(mk), _p(columns), rows, cols, n, m, v, _p(values), _p(meta), threads)
    elif dense.dtype == np.float32:
        values = np.zeros(g.n_values, np.float32)
        st = L.spatha_vnm_encode_f32(_p(dense), _p(mk), _p(columns), rows, cols, n, m, v, _p(values), _p(meta), threads)
    else:
        raise TypeError("dense must be float16 or float32")
    _lib.check(st, "spatha_vnm_encode")
    return values, meta


def decode(values, metadata, columns, rows, cols, n, m, v, threads=0):
    values = np.ascontiguousarray(values)
    metadata = np.ascontiguousarray(metadata).view(np.uint32)
    columns = np.ascontiguousarray(columns, dtype=np.uint32).reshape(-1)
    g = geometry(rows, cols, n, m, v)
    if values.size != g.n_values or metadata.size != g.n_metadata or columns.size != g.n_columns:
        raise ValueError("array sizes do not match the format geometry")
    dense = np.empty((rows, cols), values.dtype)
    L = _lib.lib()
    if values.dtype == np.float16:
        st = L.spatha_vnm_decode_f16(_p(values), _p(metadata), _p(columns), rows, cols, n, m, v, _p(dense), threads)
    elif values.dtype == np.float32:
        st = L.spatha_vnm_decode_f32(_p(values), _p(metadata), _p(columns), rows, cols, n, m, v, _p(dense), threads)
    else:
        raise TypeError("values must be float16 or float32")
    _lib.check(st, "spatha_vnm_decode")
    return dense


def select_columns(dense_abs, n, m, v, threads=0, gpu=False, stream=None, exact_ties=True):
    """|A| float32 (rows, cols) -> (masks int32 (rows, cols), columns int32).  gpu=True runs the search over the
    column subsets on the GPU (same result bit for bit; 12 s -> milliseconds for a 4096 x 1024 matrix at m = 32).
    exact_ties=False (GPU path only): among EQUAL magnitudes the lower column wins instead of the reference's
    history-dependent choice, which spares the sequential replay that such ties otherwise force."""
    d = np.ascontiguousarray(dense_abs, dtype=np.float32)
    rows, cols = d.shape
    g = geometry(rows, cols, n, m, v)
    masks = np.zeros((rows, cols), np.int32)
    columns = np.zeros(g.n_columns, np.int32)
    if gpu:
        _lib.check(_lib.lib().spatha_vnm_select_columns_f32_gpu(_p(d), rows, cols, n, m, v, _p(masks), _p(columns), threads,
                                                                1 if exact_ties else 0, stream),
                   "spatha_vnm_select_columns_f32_gpu")
    else:
        _lib.check(_lib.lib().spatha_vnm_select_columns_f32(_p(d), rows, cols, n, m, v, _p(masks), _p(columns), threads),
                   "spatha_vnm_select_columns_f32")
    return masks, columns


def random_pattern(rows, cols, n, m, v):
    """Pattern drawn from the C library's rand() stream in the reference's order."""
    g = geometry(rows, cols, n, m, v)
    meta = np.zeros(g.n_metadata, np.uint32)
    columns = np.zeros(g.n_columns, np.uint32)
    _lib.check(_lib.lib().spatha_vnm_random_pattern(rows, cols, n, m, v, _p(meta), _p(columns)),
               "spatha_vnm_random_pattern")
    return meta, columns


def fill_rand_small_ints(count):
    out = np.empty(count, np.float16)
    _lib.check(_lib.lib().spatha_fill_rand_small_ints_f16(_p(out), count), "spatha_fill_rand_small_ints_f16")
    return out


def benchmark_inputs(rows, cols, ncols_b, n, m, v):
    """(B, metadata, columns, values) of one reference benchmark run, drawn from rand() in its order."""
    g = geometry(rows, cols, n, m, v)
    B = np.empty((cols, ncols_b), np.float16)
    meta = np.zeros(g.n_metadata, np.uint32)
    columns = np.zeros(g.n_columns, np.uint32)
    vals = np.empty(g.n_values, np.float16)
    _lib.check(_lib.lib().spatha_benchmark_inputs_f16(rows, cols, ncols_b, n, m, v, _p(B), _p(meta), _p(columns), _p(vals)),
               "spatha_benchmark_inputs_f16")
    return B, meta, columns, vals


def pack_meta_blob(metadata, columns):
    metadata = np.ascontiguousarray(metadata).view(np.uint32)
    columns = np.ascontiguousarray(columns, dtype=np.uint32).reshape(-1)
    off = ctypes.c_int64()
    words = ctypes.c_int64()
    L = _lib.lib()
    _lib.check(L.spatha_vnm_pack_meta_blob(None, metadata.size, None, columns.size, None, ctypes.byref(off),
                                           ctypes.byref(words)), "spatha_vnm_pack_meta_blob")
    blob = np.zeros(words.value, np.uint32)
    _lib.check(L.spatha_vnm_pack_meta_blob(_p(metadata), metadata.size, _p(columns), columns.size, _p(blob),
                                           ctypes.byref(off), ctypes.byref(words)), "spatha_vnm_pack_meta_blob")
    return blob, off.value


def save(path, values, metadata, columns, rows, cols, n, m, v):
    """Writes an encoded matrix to the library's on-disk container (values fp16 or fp32)."""
    values = np.ascontiguousarray(values)
    metadata = np.ascontiguousarray(metadata).view(np.uint32)
    columns = np.ascontiguousarray(columns, dtype=np.uint32).reshape(-1)
    g = geometry(rows, cols, n, m, v)
    if values.size != g.n_values or metadata.size != g.n_metadata or columns.size != g.n_columns:
        raise ValueError("array sizes do not match the format geometry")
    bits = {np.dtype(np.float16): 16, np.dtype(np.float32): 32}.get(values.dtype)
    if bits is None:
        raise TypeError("values must be float16 or float32")
    _lib.check(_lib.lib().spatha_vnm_file_write(str(path).encode(), rows, cols, n, m, v, bits, _p(values), _p(metadata),
                                                _p(columns)), "spatha_vnm_file_write")


def load(path):
    """Reads a container written by `save`: (values, metadata, columns, geometry)."""
    L = _lib.lib()
    g = _lib.Geometry()
    bits = ctypes.c_int(0)
    _lib.check(L.spatha_vnm_file_info(str(path).encode(), ctypes.byref(g), ctypes.byref(bits)), "spatha_vnm_file_info")
    values = np.empty(g.n_values, np.float16 if bits.value == 16 else np.float32)
    metadata = np.empty(g.n_metadata, np.uint32)
    columns = np.empty(g.n_columns, np.uint32)
    _lib.check(L.spatha_vnm_file_read(str(path).encode(), _p(values), _p(metadata), _p(columns)), "spatha_vnm_file_read")
    return values, metadata, columns, g


def synthetic_vnm(rows, cols, n, m, v, seed=0, value_std=1.0, integer_values=False):
    """Seeded synthetic V:N:M matrix in compressed form (values fp16, metadata, columns):
    per V x m block 4 of the m columns drawn uniformly, per row 2 of those 4 kept uniformly;
    non-zeros ~ N(0, value_std) (or small integers in [-4, 4])."""
    g = geometry(rows, cols, n, m, v)
    rng = np.random.default_rng(seed)
    ngroups = g.ksp // 2
    full = cols // m
    columns = np.zeros((rows // v, ngroups, 4), np.uint32)
    if full > 0:
        keys = rng.random((rows // v, full, m))
        columns[:, :full, :] = np.sort(np.argsort(keys, axis=-1)[..., :4], axis=-1).astype(np.uint32)
    if cols % m:
        columns[:, full, :] = np.arange(4, dtype=np.uint32)
    pair_keys = rng.random((rows, ngroups, 4))
    pairs = np.sort(np.argsort(pair_keys, axis=-1)[..., :2], axis=-1).astype(np.uint32)   # (rows, ngroups, 2)
    if integer_values:
        vals = rng.integers(-4, 5, size=(rows, ngroups, 2)).astype(np.float16)
    else:
        vals = (rng.standard_normal((rows, ngroups, 2)) * value_std).astype(np.float16)
    # entries whose dense column falls outside the matrix carry zero
    dcol = (np.arange(ngroups)[None, :, None] * m +
            np.take_along_axis(columns[np.arange(rows) // v], pairs.astype(np.int64), axis=-1))
    vals[dcol >= cols] = 0
    # scatter into the storage layout (closed form)
    r = np.arange(rows)[:, None]
    gidx = np.arange(ngroups)[None, :]
    R16, q, p, s = r >> 4, (r >> 2) & 3, (r >> 1) & 1, r & 1
    t, u = gidx >> 2, gidx & 3
    vi = R16 * 16 * g.ksp + t * 128 + q * 32 + u * 8 + p * 4 + s * 2
    values = np.zeros(g.n_values, np.float16)
    values[vi.reshape(-1)] = vals[..., 0].reshape(-1)
    values[vi.reshape(-1) + 1] = vals[..., 1].reshape(-1)
    wi = (r >> 5) * (g.ksp >> 3) * 16 + t * 16 + ((r >> 4) & 1) * 8 + q * 2 + p
    nib = (pairs[..., 0] | (pairs[..., 1] << 2)).astype(np.uint32) << (s * 16 + u * 4).astype(np.uint32)
    meta = np.zeros(g.n_metadata, np.uint32)
    np.bitwise_or.at(meta, wi.reshape(-1), nib.reshape(-1))
    return values, meta, columns.reshape(-1)
