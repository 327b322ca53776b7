"""Seeded random shapes through the library's AUTOMATIC kernel choice, bit-exact against the CPU oracle.

The fixed cases of test_spmm_gpu.py name their shapes; the rules of the automatic choice (tile counts against the number
of CUs, k-steps per tile, V class, m, layout, fused write-out) have boundaries where no fixed case sits, and some of the
kernels behind them load registers asynchronously, which only results can check.  Here ~200 shapes are drawn so that
every class of rule is reached: integer-valued operands (fp32 accumulation exact, so the result must equal the oracle's
bit for bit), row-major / transposed + bias / fused bias, ragged N and K.  The shape and the kernel's name are printed
before each launch; the first mismatch stops the sweep."""
import collections

import numpy as np
import pytest
import torch

import oracle
from venom_amd import format as F
from venom_amd import spatha

V_CHOICES = [32, 64, 96, 128, 192, 256]
M_CHOICES = [4, 5, 7, 8, 10, 12, 16, 20, 32, 40]
STEP_CHOICES = [1, 2, 3, 4, 6, 8, 12, 16, 24, 33, 41]
N_SMALL = [8, 16, 24, 32, 40, 48, 56, 64, 72, 104, 128, 136, 200, 256, 264, 520, 1032]
# (rows, N) pairs whose tile counts reach the rules that ask for one or more whole rounds of the CUs (256 on MI355X)
BIG_GRIDS = [(4096, 12288), (2048, 16384), (1024, 16384), (512, 8192), (4096, 4096), (1024, 4096), (1024, 8200), (1536, 4104),
             (3072, 2048), (512, 16384), (2048, 4096), (1024, 2048), (768, 8192), (6144, 2048)]
MAX_WORK = 6e9          # rows * N * Ksp per case: bounds the oracle's time (about 0.1 s with all host cores)
MODES = ["row_major", "transposed_bias", "fused_bias_row_major", "fused_bias_transposed"]


def draw_cases(count, seed=20240):
    """Deterministic list of (rows, cols, N, m, v, mode).  Every second case takes its (rows, N) from BIG_GRIDS (rounded
    to the drawn V) with few k-steps; the others are small and ragged."""
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        v = int(rng.choice(V_CHOICES))
        m = int(rng.choice(M_CHOICES))
        steps = int(rng.choice(STEP_CHOICES))
        if len(cases) % 2 == 0:
            rows, N = BIG_GRIDS[int(rng.integers(len(BIG_GRIDS)))]
            rows = max(v, rows // v * v)
            if rng.random() < 0.3:
                N += 8 * int(rng.integers(1, 16))
        else:
            rows = v * int(rng.integers(1, max(2, 1536 // v) + 1))
            N = int(rng.choice(N_SMALL))
        # k-steps of 32 stored values = 16 groups of m columns; a ragged tail in half of the cases
        cols = steps * 16 * m
        if rng.random() < 0.5:
            cols -= int(rng.integers(1, m + 4))
        cols = max(cols, m)
        ksp = F.geometry(rows, cols, 2, m, v).ksp
        while rows * N * ksp > MAX_WORK and steps > 1:
            steps = max(1, steps // 2)
            cols = steps * 16 * m
            ksp = F.geometry(rows, cols, 2, m, v).ksp
        if rows * N * ksp > MAX_WORK:
            continue
        cases.append((rows, cols, N, m, v, MODES[int(rng.integers(len(MODES)))]))
    return cases


def test_drawn_cases_are_representable():
    cases = draw_cases(200)
    assert len(cases) == 200 and len(set(cases)) > 190
    for rows, cols, N, m, v, mode in cases:
        g = F.geometry(rows, cols, 2, m, v)           # raises for a shape the format cannot hold
        assert N % 8 == 0 and rows % v == 0 and rows * N * g.ksp <= MAX_WORK
    assert {c[4] for c in cases} == set(V_CHOICES) and {c[3] for c in cases} == set(M_CHOICES)
    assert {c[5] for c in cases} == set(MODES)


def _dev(a, gpu):
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(np.ascontiguousarray(a)).to(gpu)


KERNELS_REACHED = collections.Counter()


@pytest.mark.gpu
@pytest.mark.parametrize("chunk", range(4))
def test_automatic_choice_on_random_shapes_bit_exact(gpu, chunk):
    cases = draw_cases(200)
    kernels = KERNELS_REACHED
    for i, (rows, cols, N, m, v, mode) in enumerate(cases):
        if i // 50 != chunk:
            continue
        transposed = mode in ("transposed_bias", "fused_bias_transposed")
        fused = mode.startswith("fused")
        vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=1000 + i, integer_values=True)
        rng = np.random.default_rng(i)
        B = rng.integers(-4, 5, size=(cols, N)).astype(np.float16)
        bias = None if mode == "row_major" else rng.integers(-8, 9, size=rows).astype(np.float16)
        plan = spatha.SpmmPlan(_dev(vals, gpu), _dev(meta, gpu), _dev(columns, gpu), rows, cols, 2, m, v)
        name = plan.kernel_name(N, 1 if transposed else 0, 0)
        print("case %d: %d x %d x %d, %d:2:%d, %s -> %s" % (i, rows, cols, N, v, m, mode, name), flush=True)
        assert name is not None
        got = plan.run(_dev(B, gpu), bias=None if bias is None else _dev(bias, gpu), transposed_out=transposed,
                       activation="none" if fused else None)
        torch.cuda.synchronize()
        got = got.cpu().numpy()
        want = oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B, bias=bias, transposed_out=True) if bias is not None \
            else oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B)
        if bias is not None and not transposed:
            want = np.ascontiguousarray(want.T)
        if not np.array_equal(got.view(np.uint16), want.view(np.uint16)):
            bad = np.argwhere(got.view(np.uint16) != want.view(np.uint16))
            pytest.fail("case %d (%d x %d x %d, %d:2:%d, %s, kernel %s): %d entries differ, first at %s: got %r, want %r"
                        % (i, rows, cols, N, v, m, mode, name, len(bad), tuple(bad[0]), got[tuple(bad[0])], want[tuple(bad[0])]))
        kernels[name.split("+")[0]] += 1
        del plan
    print("kernels reached so far:", dict(kernels), flush=True)
    if chunk == 3 and sum(kernels.values()) > 150:
        assert len(kernels) >= 12          # the sweep is only worth its time if it reaches most of the registry


@pytest.mark.gpu
def test_every_kernel_id_on_random_shapes_bit_exact(gpu):
    """The same draw with another seed, through EVERY kernel id that accepts the shape (a caller may name an id, and
    spatha_spmm_tune runs them all): 120 shapes, about 900 launches, each equal to the oracle bit for bit."""
    launches = 0
    reached = set()
    for i, (rows, cols, N, m, v, mode) in enumerate(draw_cases(120, seed=11)):
        transposed = mode in ("transposed_bias", "fused_bias_transposed")
        fused = mode.startswith("fused")
        vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=5000 + i, integer_values=True)
        rng = np.random.default_rng(7000 + i)
        B = rng.integers(-4, 5, size=(cols, N)).astype(np.float16)
        bias = None if mode == "row_major" else rng.integers(-8, 9, size=rows).astype(np.float16)
        want = oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B, bias=bias, transposed_out=True) if bias is not None \
            else oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B)
        if bias is not None and not transposed:
            want = np.ascontiguousarray(want.T)
        plan = spatha.SpmmPlan(_dev(vals, gpu), _dev(meta, gpu), _dev(columns, gpu), rows, cols, 2, m, v)
        dB, dbias = _dev(B, gpu), None if bias is None else _dev(bias, gpu)
        for variant in range(1, spatha.num_variants()):
            name = plan.kernel_name(N, 1 if transposed else 0, variant)
            if name is None:
                continue
            print("case %d id %d: %d x %d x %d, %d:2:%d, %s -> %s" % (i, variant, rows, cols, N, v, m, mode, name), flush=True)
            try:
                got = plan.run(dB, bias=dbias, transposed_out=transposed, activation="none" if fused else None, variant=variant)
            except RuntimeError as e:
                assert fused and "no kernel" in str(e), (variant, str(e))    # ids without a fused write-out say so
                continue
            torch.cuda.synchronize()
            got = got.cpu().numpy()
            if not np.array_equal(got.view(np.uint16), want.view(np.uint16)):
                bad = np.argwhere(got.view(np.uint16) != want.view(np.uint16))
                pytest.fail("case %d id %d (%d x %d x %d, %d:2:%d, %s, kernel %s): %d entries differ, first at %s"
                            % (i, variant, rows, cols, N, v, m, mode, name, len(bad), tuple(bad[0])))
            launches += 1
            reached.add(variant)
        del plan
    print("launches", launches, "ids", sorted(reached), flush=True)
    assert launches > 600 and len(reached) >= 20
