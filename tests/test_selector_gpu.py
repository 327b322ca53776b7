"""The magnitude selector with its search phase on the GPU (spatha_vnm_select_columns_f32_gpu) against the oracle, the
host library and the vectors written by the reference's own selector: masks and column offsets must be identical,
ties (which depend on the reference's permutation history), all-zero blocks and narrow tails included."""
import time

import numpy as np
import pytest

import oracle
from helpers import golden_cases
from venom_amd import format as F

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("path", [p for p in golden_cases() if "fixed" not in p], ids=lambda p: p.split("vnm_")[-1][:-4])
def test_gpu_search_matches_reference_vectors(gpu, path):
    z = np.load(path)
    d, n, m, v = z["dense"], int(z["n"]), int(z["m"]), int(z["v"])
    masks, columns = F.select_columns(np.abs(d), n, m, v, gpu=True)
    assert np.array_equal(masks, z["masks"])
    assert np.array_equal(columns, z["columns"])


@pytest.mark.parametrize("rows,cols,m,v", [(64, 64, 8, 32), (64, 67, 8, 32), (64, 70, 8, 32), (128, 66, 8, 64),
                                           (64, 64, 16, 32), (32, 64, 32, 32), (64, 32, 4, 32), (128, 100, 20, 128),
                                           (64, 75, 10, 32), (128, 100, 48, 128), (192, 40, 40, 64)])
@pytest.mark.parametrize("kind", ["gauss", "ties", "sparse"])
def test_gpu_search_equals_oracle(gpu, rows, cols, m, v, kind):
    rng = np.random.default_rng(rows + cols * 3 + m)
    if kind == "gauss":
        d = np.abs(rng.standard_normal((rows, cols))).astype(np.float32)
    elif kind == "ties":
        d = rng.integers(0, 3, size=(rows, cols)).astype(np.float32)
    else:
        d = np.abs(rng.standard_normal((rows, cols))).astype(np.float32) * (rng.random((rows, cols)) < 0.3)
        d[:, :m] = 0
    masks, columns = F.select_columns(d, 2, m, v, gpu=True)
    if m <= 32:
        omasks, ocolumns = oracle.select_columns(d, 2, m, v)
    else:       # the oracle's loop nest takes minutes from m = 40 on: the host library (itself checked against it) stands in
        omasks, ocolumns = F.select_columns(d, 2, m, v)
    assert np.array_equal(columns, ocolumns)
    assert np.array_equal(masks, omasks)


def test_gpu_search_on_a_bert_large_ffn_weight(gpu):
    """4096 x 1024 at 64:2:32: 35 960 subsets for each of 2048 blocks.  Same answer as the host search, far sooner."""
    import torch

    from venom_amd.grouped_nmv_tensor import nm_vector_mask_sparsify

    torch.manual_seed(0)
    w = torch.randn(4096, 1024) * 0.02
    t0 = time.perf_counter()
    gm, gc = nm_vector_mask_sparsify(w, 2, 32, 64, gpu=True)
    t_gpu = time.perf_counter() - t0
    # the host search on a slice of the rows (the whole matrix takes ~10 s on 16 cores)
    hm, hc = nm_vector_mask_sparsify(w[:512], 2, 32, 64, gpu=False)
    assert torch.equal(gm[:512], hm) and torch.equal(gc[:hc.numel()], hc)
    assert gm.sum().item() == 4096 * (1024 // 32) * 2
    print("GPU-assisted selector, 4096 x 1024 at 64:2:32: %.2f s" % t_gpu)
    assert t_gpu < 5.0


def test_without_tie_replay_equal_magnitudes_go_to_the_lower_column(gpu):
    """exact_ties=False: same column offsets, and per row the two largest of the four chosen columns with the lower
    column winning among equals; identical to the exact result wherever no tie decides."""
    rng = np.random.default_rng(3)
    rows, cols, m, v = 128, 128, 8, 64
    d = rng.integers(0, 4, size=(rows, cols)).astype(np.float32)          # plenty of equal magnitudes
    exact_masks, exact_cols = F.select_columns(d, 2, m, v, gpu=True)
    masks, columns = F.select_columns(d, 2, m, v, gpu=True, exact_ties=False)
    assert np.array_equal(columns, exact_cols)
    ngroups = cols // m
    chosen = columns.reshape(rows // v, -1, 4)[:, :ngroups]
    for r in range(rows):
        for g in range(ngroups):
            c = chosen[r // v, g]
            x = d[r, g * m + c]
            order = sorted(range(4), key=lambda i: (-x[i], i))[:2]        # largest first, lower index among equals
            want = np.zeros(m, np.int32)
            if d[(r // v) * v:(r // v + 1) * v, g * m:(g + 1) * m].any():
                want[c[order]] = 1
            assert np.array_equal(masks[r, g * m:(g + 1) * m], want), (r, g)
            kept, kept_exact = np.sort(d[r, g * m:(g + 1) * m][masks[r, g * m:(g + 1) * m] == 1]), \
                np.sort(d[r, g * m:(g + 1) * m][exact_masks[r, g * m:(g + 1) * m] == 1])
            assert np.array_equal(kept, kept_exact)                          # the same magnitudes either way
    g2 = np.abs(rng.standard_normal((rows, cols))).astype(np.float32)     # no ties: the two settings agree exactly
    a = F.select_columns(g2, 2, m, v, gpu=True)
    b = F.select_columns(g2, 2, m, v, gpu=True, exact_ties=False)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
