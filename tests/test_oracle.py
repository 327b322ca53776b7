"""Pins the CPU oracle: golden vectors written by the reference's own Python host code,
closed-form layout maps, brute force on tiny inputs, numpy for the arithmetic."""
import itertools
import os

import numpy as np
import pytest

import oracle
from helpers import rel_err, golden_cases, ksp_of, numpy_decode, random_conforming, slot_maps


@pytest.mark.parametrize("path", golden_cases(), ids=lambda p: p.split("vnm_")[-1][:-4])
def test_oracle_matches_reference_vectors(path):
    z = np.load(path)
    d, n, m, v = z["dense"], int(z["n"]), int(z["m"]), int(z["v"])
    rows, cols = d.shape
    s = oracle.sizes(rows, cols, n, m, v)
    assert s["ksp"] == int(z["ksp"])
    assert s["n_values"] == z["values"].size and s["n_metadata"] == z["metadata"].size
    assert s["n_columns"] == z["columns"].size
    if "fixed" not in path:
        masks, columns = oracle.select_columns(np.abs(d), n, m, v)
        assert np.array_equal(masks, z["masks"])
        assert np.array_equal(columns, z["columns"])
    if bool(z["encode_defined"]):
        vals, meta = oracle.encode(d * z["masks"], z["columns"].astype(np.uint32), n, m, v, mask=z["masks"])
        assert np.array_equal(vals, z["values"])
        assert np.array_equal(meta, z["metadata"].view(np.uint32))
        back = oracle.decode(z["values"], z["metadata"].view(np.uint32), z["columns"].astype(np.uint32), rows, cols, n, m, v)
        assert np.array_equal(back, z["decoded"])


@pytest.mark.parametrize("rows,cols,m,v", [(64, 64, 8, 32), (128, 96, 8, 64), (128, 256, 16, 128), (64, 40, 4, 32),
                                           (64, 70, 8, 32), (256, 512, 32, 128)])
def test_oracle_layout_is_the_closed_form(rows, cols, m, v):
    dense, mask, columns = random_conforming(rows, cols, 2, m, v, seed=rows + cols + m)
    vals, meta = oracle.encode(dense, columns, 2, m, v)                # non-zero driven
    vals2, meta2 = oracle.encode(dense, columns, 2, m, v, mask=mask)   # mask driven
    assert np.array_equal(vals, vals2) and np.array_equal(meta, meta2)
    # the closed-form reader recovers the matrix from the oracle's arrays
    assert np.array_equal(numpy_decode(vals, meta, columns, rows, cols, 2, m, v), dense)
    assert np.array_equal(oracle.decode(vals, meta, columns, rows, cols, 2, m, v), dense)
    # the slot maps are bijections onto the arrays
    ksp = ksp_of(cols, 2, m)
    vi, wi, sh = slot_maps(rows, ksp)
    allv = np.concatenate([vi.reshape(-1), vi.reshape(-1) + 1])
    assert np.array_equal(np.sort(allv), np.arange(rows * ksp))
    slots = wi.reshape(-1) * 8 + sh.reshape(-1) // 4
    assert np.array_equal(np.sort(slots), np.arange(rows // 2 * (ksp // 8) * 8))


def test_half_conversion_against_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.half_to_float(bits)
    ref = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(f.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * s for s in (1e-8, 1e-5, 1e-3, 1.0, 300.0, 7e4)])
    # exact ties and boundaries
    x = np.concatenate([x, np.array([65504, 65519.99, 65520, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 0.0, -0.0,
                                     1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11, np.inf, -np.inf], np.float32)])
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.float_to_half(x), x.astype(np.float16).view(np.uint16))
    a = rng.integers(0, 0x7C00, 100000).astype(np.uint16) | (rng.integers(0, 2, 100000).astype(np.uint16) << 15)
    b = rng.integers(0, 0x7C00, 100000).astype(np.uint16) | (rng.integers(0, 2, 100000).astype(np.uint16) << 15)
    exact = a.view(np.float16).astype(np.float64) + b.view(np.float16).astype(np.float64)
    with np.errstate(over="ignore"):
        want = exact.astype(np.float16)     # one rounding from the exact sum
    assert np.array_equal(oracle.add_half(a, b), want.view(np.uint16))


def _brute_select(block, n, m):
    """argmax over ascending 4-subsets of sum over rows of the n largest, first maximum wins."""
    best, best_q = 0.0, None
    for q in itertools.combinations(range(m), 4):
        sub = block[:, q].astype(np.float64)
        tot = np.sort(sub, axis=1)[:, -n:].sum()
        if tot > best * (1 + 1e-12) and tot > best:
            best, best_q = tot, q
    return best_q


def test_selector_brute_force_small():
    rng = np.random.default_rng(5)
    rows, cols, n, m, v = 64, 48, 2, 8, 32
    d = np.abs(rng.standard_normal((rows, cols))).astype(np.float32)
    masks, columns = oracle.select_columns(d, n, m, v)
    ksp = ksp_of(cols, n, m)
    columns = columns.reshape(rows // v, ksp // 2, 4)
    for b in range(rows // v):
        for g in range(cols // m):
            blk = d[b * v:(b + 1) * v, g * m:(g + 1) * m]
            q = _brute_select(blk, n, m)
            assert tuple(columns[b, g]) == q
            mk = masks[b * v:(b + 1) * v, g * m:(g + 1) * m]
            assert (mk.sum(axis=1) == n).all()
            assert mk[:, [c for c in range(m) if c not in q]].sum() == 0
            # kept entries are the n largest of the chosen four
            for r in range(v):
                kept = np.sort(blk[r][mk[r] == 1])
                assert np.array_equal(kept, np.sort(blk[r, list(q)])[-n:])


def test_selector_dominant_quadruple_closed_form():
    # row class k keeps its two large entries in columns q[k], q[k+1]: only the quadruple q
    # collects every large entry, so it must win, and the mask must mark exactly those two.
    rows, cols, n, m, v = 32, 32, 2, 16, 32
    d = np.full((rows, cols), 0.01, np.float32)
    want = [(1, 5, 6, 14), (0, 2, 3, 15)]
    for g, q in enumerate(want):
        for r in range(rows):
            d[r, g * m + q[r % 4]] = 2.0
            d[r, g * m + q[(r + 1) % 4]] = 1.0
    masks, columns = oracle.select_columns(d, n, m, v)
    assert [tuple(x) for x in columns.reshape(-1, 4)[:2]] == want
    assert np.array_equal(masks, (d > 0.5).astype(np.int32))


def test_spmm_matches_dense_product_of_decode():
    rows, cols, N, m, v = 128, 192, 40, 8, 64
    rng = np.random.default_rng(3)
    dense, mask, columns = random_conforming(rows, cols, 2, m, v, seed=9, integer=True, dtype=np.float16)
    vals, meta = oracle.encode(dense, columns, 2, m, v)
    B = rng.integers(-4, 5, size=(cols, N)).astype(np.float16)
    want = (dense.astype(np.float64) @ B.astype(np.float64))
    got = oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B)
    assert np.array_equal(got.astype(np.float64), want)          # small integers: exact
    assert np.array_equal(oracle.dense_gemm(dense, B).astype(np.float64), want)
    bias = rng.integers(-3, 4, size=rows).astype(np.float16)
    got_t = oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B, bias=bias, transposed_out=True)
    assert np.array_equal(got_t.astype(np.float64), want.T + bias.astype(np.float64)[None, :])
    # gaussian data: within fp16 rounding of the float64 product
    dense, mask, columns = random_conforming(rows, cols, 2, m, v, seed=10, dtype=np.float16)
    vals, meta = oracle.encode(dense, columns, 2, m, v)
    B = rng.uniform(-1, 1, size=(cols, N)).astype(np.float16)
    want = dense.astype(np.float64) @ B.astype(np.float64)
    got = oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B).astype(np.float64)
    assert rel_err(got, want) < 1e-3            # one fp16 rounding (4.9e-4) of the fp32 sum
    assert oracle.check_results(got.astype(np.float16), want.astype(np.float16)) == 0
    bad = want.astype(np.float16).copy()
    bad[3, 4] += np.float16(2.0)
    assert oracle.check_results(bad, want.astype(np.float16)) == 1


def test_random_mask_invariants():
    oracle.srand(1)
    rows, cols, n, m, v = 128, 136, 2, 8, 64        # 17 groups: one full tile of 4... plus a ragged tail
    meta, columns = oracle.random_mask(rows, cols, n, m, v)
    ksp = ksp_of(cols, n, m)
    cq = columns.reshape(rows // v, ksp // 2, 4)
    full = cols // m
    assert (np.diff(cq[:, :full].astype(int), axis=-1) > 0).all() and cq[:, :full].max() < m
    assert (cq[:, full:] == 0).all()                 # cols % m == 0: nothing after the full groups
    _, wi, sh = slot_maps(rows, ksp)
    nib = (meta[wi] >> sh.astype(np.uint32)) & 0xF
    lo, hi = nib & 3, nib >> 2
    full_tiles = (full // 4) * 4
    assert (lo[:, :full_tiles] < hi[:, :full_tiles]).all()
    assert (nib[:, full_tiles:] == 0).all()          # partial last tile stays zero when m divides cols


# --- the random pattern generator's stream (src/format/format_sr_nm.cpp:151-237) ---------------------------------

def _kat_module():
    import importlib.util
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "make_random_mask_kat.py")
    spec = importlib.util.spec_from_file_location("make_random_mask_kat", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_python_restatement_of_glibc_rand_equals_the_c_library():
    """The known answers below rest on a pure-Python restatement of glibc's rand(); it must reproduce the C library's
    stream after srand(1), which is also the stream of a process that never seeds (the reference never does)."""
    import ctypes
    libc = ctypes.CDLL(None)
    libc.srand(1)
    want = [libc.rand() for _ in range(5000)]
    assert _kat_module().glibc_rand_stream(1, 5000) == want
    assert want[:3] == [1804289383, 846930886, 1681692777]


def test_shuffle_equals_libstdcxx_random_shuffle(tmp_path):
    """The oracle's shuffle and the Python one against the real std::random_shuffle (removed in C++17, so a C++14
    snippet built here), on arrays that persist from call to call as the generator's do."""
    import subprocess
    src = tmp_path / "rs.cpp"
    src.write_text("""
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>
int main() {
    std::srand(1);
    std::vector<unsigned> a{0, 1, 2, 3}, b{0, 1, 2, 3, 4, 5, 6, 7};
    for (int t = 0; t < 200; t++) {
        std::random_shuffle(a.begin(), a.end());
        std::sort(a.begin(), a.begin() + 2);
        for (unsigned x : a) std::printf("%u ", x);
        std::random_shuffle(b.begin(), b.end());
        std::sort(b.begin(), b.begin() + 4);
        for (unsigned x : b) std::printf("%u ", x);
        std::printf("\\n");
    }
    return 0;
}
""")
    exe = tmp_path / "rs"
    subprocess.check_call(["g++", "-std=c++14", "-O1", "-Wno-deprecated-declarations", "-o", str(exe), str(src)])
    want = [[int(x) for x in line.split()] for line in subprocess.check_output([str(exe)]).decode().splitlines()]
    assert len(want) == 200
    oracle.srand(1)
    a, b = np.arange(4, dtype=np.uint32), np.arange(8, dtype=np.uint32)
    stream = _kat_module().Stream(1)
    pa, pb = [0, 1, 2, 3], list(range(8))
    for row in want:
        a = oracle.shuffle(a); a[:2] = np.sort(a[:2])
        b = oracle.shuffle(b); b[:4] = np.sort(b[:4])
        stream.shuffle(pa); pa[:2] = sorted(pa[:2])
        stream.shuffle(pb); pb[:4] = sorted(pb[:4])
        assert list(a) + list(b) == row and pa + pb == row


def test_random_mask_known_answers():
    """32 x 32, 2:8, V = 32, first matrix of a process (stream position 0).  Hand walk of the first word
    (format_sr_nm.cpp:157-177; glibc rand() after srand(1) = 1804289383, 846930886, 1681692777, 1714636915, 1957747793,
    424238335, 719885386, 1649760492, 596516649, ...; a shuffle of {a0..a3} swaps a1 with a[r % 2], a2 with a[r % 3],
    a3 with a[r % 4]):
      group 0: {0,1,2,3}: 1804289383 % 2 = 1 (no swap), 846930886 % 3 = 1 -> {0,2,1,3}, 1681692777 % 4 = 1 -> {0,3,1,2};
               first two sorted = (0, 3) -> bits 0b1100 = 0xC
      group 1: {0,3,1,2}: 1714636915 % 2 = 1, 1957747793 % 3 = 2, 424238335 % 4 = 3: no swap; pair (0, 3) -> 0xC
      group 2: {0,3,1,2}: 719885386 % 2 = 0 -> {3,0,1,2}, 1649760492 % 3 = 0 -> {1,0,3,2}, 596516649 % 4 = 1 -> {1,2,3,0};
               pair (1, 2) -> 1 | 2 << 2 = 0x9
    so the word ends in ...9CC, and 16 words x 8 groups x 3 draws = 384 draws precede the column-loc draws
    (:213-229), whose first shuffle of {0..7} uses draws 384..390 and leaves (1, 3, 4, 5) in front."""
    oracle.srand(1)
    meta, columns = oracle.random_mask(32, 32, 2, 8, 32)
    assert [hex(int(w)) for w in meta[:4]] == ["0xd89e99cc", "0xcdc9dd4d", "0xed8ed4c9", "0x9c448ee9"]
    assert int(meta[15]) == 0xEDC494E9 and not meta[16:].any()       # the second tile of the padded row stays zero
    assert columns.reshape(-1, 4)[:4].tolist() == [[1, 3, 4, 5], [1, 3, 4, 6], [1, 3, 4, 6], [1, 5, 6, 7]]
    assert not columns.reshape(-1, 4)[4:].any()


def test_random_mask_stream_over_consecutive_matrices():
    """Five matrices drawn one after another from one stream (complete tiles, complete groups beyond the last tile,
    K % m != 0 tails, m = 16, plain 2:4, several 32-row and V-row blocks) against answers derived without the oracle
    (tests/golden/make_random_mask_kat.py)."""
    import json
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "random_mask_kat.json")) as f:
        kat = json.load(f)
    assert len(kat) == 5
    oracle.srand(1)
    for c in kat:
        meta, columns = oracle.random_mask(c["rows"], c["cols"], 2, c["m"], c["v"])
        assert np.array_equal(meta, np.array(c["metadata"], np.uint32)), c["rows"]
        assert np.array_equal(columns, np.array(c["columns"], np.uint32)), c["rows"]
    # the stream has advanced by exactly the number of draws the walk counts
    import ctypes
    libc = ctypes.CDLL(None)
    libc.srand(1)
    for _ in range(kat[-1]["draws_after"]):
        libc.rand()
    want_next = libc.rand()
    oracle.srand(1)
    for c in kat:
        oracle.random_mask(c["rows"], c["cols"], 2, c["m"], c["v"])
    assert oracle.lib().vo_rand() == want_next
