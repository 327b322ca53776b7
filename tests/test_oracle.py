"""Pins the CPU oracle: golden vectors written by the reference's own Python host code,
closed-form layout maps, brute force on tiny inputs, numpy for the arithmetic."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import golden_cases, ksp_of, numpy_decode, random_conforming, slot_maps


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
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1.0)) < 2e-3
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
