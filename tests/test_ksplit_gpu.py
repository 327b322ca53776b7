"""k-loops split over several workgroups (`spatha_spmm_run_ws`, a run that brings a workspace) against the CPU oracle, bit for bit
on integer-valued operands: few tiles with long k-loops (every tile in 2, 3 or 4 parts), the two kernels that have the hand-over
(128 x 128 tiles, 128 x 256 tiles with tall consumer blocks), both layouts, bias, fused bias.  Shapes are sized for the 256 CUs of
an MI355X."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from venom_amd import _lib
from venom_amd import format as F
from venom_amd import spatha

pytestmark = pytest.mark.gpu


def _dev(a, gpu):
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(np.ascontiguousarray(a)).to(gpu)


SPLIT_CASES = [
    # rows, cols, N, m, v, transposed, tile width of the kernel that runs split, tiles that run split, parts per tile
    (512, 16384, 1024, 8, 128, False, 128, 32, 4),      # 32 tiles of 128 k-steps on 256 CUs: four parts of 32
    (1024, 24576, 2048, 16, 128, False, 128, 128, 2),   # 128 tiles of 96 k-steps: two parts of 48
    (512, 16384, 1032, 8, 128, True, 128, 36, 4),       # transposed + bias, ragged N
    (512, 32768, 1024, 16, 128, True, 256, 16, 4),      # transposed + bias, 128 x 256 tiles with tall consumer blocks
    (768, 24560, 520, 12, 256, False, 128, 30, 4),      # V = 256, K tail, ragged N
    (384, 12288, 256, 8, 128, False, 128, 6, 3),        # six tiles of 96 k-steps: three parts of 32 (four would leave 24)
]


def _operands(rows, cols, N, m, v, with_bias, gpu):
    vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=rows + N, integer_values=True)
    rng = np.random.default_rng(N + m)
    B = rng.integers(-4, 5, size=(cols, N), dtype=np.int8).astype(np.float16)
    bias = rng.integers(-8, 9, size=rows).astype(np.float16) if with_bias else None
    plan = spatha.SpmmPlan(_dev(vals, gpu), _dev(meta, gpu), _dev(columns, gpu), rows, cols, 2, m, v)
    return vals, meta, columns, B, bias, plan


def _workspace(need, tickets, gpu):
    """A workspace cleared once through the library (poisoned before that); only the tickets have to be zero, the partial
    sums are written before they are read."""
    ws = torch.full((need,), 0xAB, dtype=torch.uint8, device=gpu)
    _lib.check(_lib.lib().spatha_spmm_workspace_init(ws.data_ptr(), need, None), "workspace_init")
    ws[tickets:].fill_(0xAB)
    return ws


@pytest.mark.parametrize("rows,cols,N,m,v,transposed,bn,split_tiles,parts", SPLIT_CASES)
@pytest.mark.parametrize("fused_bias", [False, True])
def test_split_runs_equal_the_oracle(gpu, rows, cols, N, m, v, transposed, bn, split_tiles, parts, fused_bias):
    print("k-split case", rows, cols, N, m, v, transposed, bn, split_tiles, parts, fused_bias, flush=True)
    if torch.cuda.get_device_properties(gpu).multi_processor_count != 256:
        pytest.skip("the cases are sized for 256 compute units")
    vals, meta, columns, B, bias, plan = _operands(rows, cols, N, m, v, transposed or fused_bias, gpu)
    fused = bias is not None and not transposed
    need = plan.workspace_bytes(N, transposed, fused)
    # one ticket per 64 x 64 block (rounded up to 256 bytes) + fp32 partial tiles: this pins which tiles run in how many parts
    tickets = -(-(split_tiles * 2 * (bn // 64) * 4) // 256) * 256
    assert need == tickets + split_tiles * parts * 128 * bn * 4
    want = oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B, bias=bias, transposed_out=True) if bias is not None \
        else oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B)
    if bias is not None and not transposed:
        want = np.ascontiguousarray(want.T)
    dB = _dev(B, gpu)
    dbias = None if bias is None else _dev(bias, gpu)
    act = "none" if fused else None
    ws = _workspace(need, tickets, gpu)
    out = torch.full((N, rows) if transposed else (rows, N), float("nan"), dtype=torch.float16, device=gpu)
    for rep in range(3):            # later calls find the tickets as the earlier ones left them (zero again)
        plan.run(dB, bias=dbias, transposed_out=transposed, activation=act, split=True, workspace=ws, out=out)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16)), rep
        out.fill_(float("nan"))
    assert bool((ws[:tickets] == 0).all())
    # the plan's own workspace (kept per stream)
    got = plan.run(dB, bias=dbias, transposed_out=transposed, activation=act, split=True)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # with a workspace that is too small the same call runs unsplit, same numbers
    small = torch.zeros(1024, dtype=torch.uint8, device=gpu)
    got = plan.run(dB, bias=dbias, transposed_out=transposed, activation=act, split=True, workspace=small)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # and the ordinary entry point agrees bit for bit (integer-valued operands)
    plain = plan.run(dB, bias=dbias, transposed_out=transposed, activation=act)
    torch.cuda.synchronize()
    assert np.array_equal(plain.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_operator_splits_with_its_own_workspace(gpu):
    """`spatha.spmm` / `spatha.spmm_fused` (the PyTorch extension) keep a workspace per stream and split where the library would:
    few tokens against a long k-loop, on two streams at once, each result equal to the oracle."""
    if torch.cuda.get_device_properties(gpu).multi_processor_count != 256:
        pytest.skip("the case is sized for 256 compute units")
    rows, cols, N, m, v = 512, 16384, 1024, 8, 128
    vals, meta, columns, B, bias, plan = _operands(rows, cols, N, m, v, True, gpu)
    assert plan.workspace_bytes(N, True) > 0 and plan.workspace_bytes(N, False, True) > 0
    want_t = oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B, bias=bias, transposed_out=True)
    dv, dm, dc, dB, dbias = _dev(vals, gpu), _dev(meta, gpu), _dev(columns, gpu), _dev(B, gpu), _dev(bias, gpu)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=gpu) for _ in range(2)]
    outs = [None, None]
    for rep in range(5):
        for k in range(2):
            with torch.cuda.stream(streams[k]):
                outs[k] = spatha.spmm(dm, dc, dv, dB, dbias, rows, cols, N, v, 2, m) if k == 0 else \
                    spatha.spmm_fused(dm, dc, dv, dB, dbias, rows, cols, v, 2, m)
    torch.cuda.synchronize()
    assert np.array_equal(outs[0].cpu().numpy().view(np.uint16), want_t.view(np.uint16))
    assert np.array_equal(outs[1].cpu().numpy().view(np.uint16), np.ascontiguousarray(want_t.T).view(np.uint16))
    spatha.clear_plan_cache()


def test_shapes_with_enough_tiles_ask_for_no_workspace(gpu):
    rows, cols, m, v = 4096, 1024, 8, 64
    vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=1, integer_values=True)
    plan = spatha.SpmmPlan(_dev(vals, gpu), _dev(meta, gpu), _dev(columns, gpu), rows, cols, 2, m, v)
    assert plan.workspace_bytes(16384) == 0 and plan.workspace_bytes(16384, True) == 0
    B = np.random.default_rng(1).integers(-4, 5, size=(cols, 256)).astype(np.float16)
    a = plan.run(_dev(B, gpu), split=True)
    b = plan.run(_dev(B, gpu))
    assert torch.equal(a, b)
    L = _lib.lib()
    assert L.spatha_spmm_workspace_bytes(None, 256, 0, 0) == 0
    assert L.spatha_spmm_workspace_bytes(plan._handle, 12, 0, 0) == 0        # N % 8


def test_split_gaussian_within_tolerance_and_deterministic(gpu):
    """Gaussian operands: the parts' sums are added in part order whatever part finishes last, so two runs give the same bits, and
    the result stays within the tolerance of the float64 product."""
    import sys, os
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from helpers import rel_err
    if torch.cuda.get_device_properties(gpu).multi_processor_count != 256:
        pytest.skip("the case is sized for 256 compute units")
    rows, cols, N, m, v = 1024, 16384, 1024, 8, 128
    vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=0, value_std=1.0)
    B = np.random.default_rng(0).uniform(-1, 1, size=(cols, N)).astype(np.float16)
    plan = spatha.SpmmPlan(_dev(vals, gpu), _dev(meta, gpu), _dev(columns, gpu), rows, cols, 2, m, v)
    assert plan.workspace_bytes(N) > 0
    dB = _dev(B, gpu)
    runs = [plan.run(dB, split=True).cpu().numpy() for _ in range(4)]
    for r in runs[1:]:
        assert np.array_equal(r.view(np.uint16), runs[0].view(np.uint16))
    exact = oracle.decode(vals, meta, columns, rows, cols, 2, m, v).astype(np.float64) @ B.astype(np.float64)
    e = rel_err(runs[0], exact)
    print("k-split, Gaussian: max rel err %.3e" % e, flush=True)
    assert e <= 1e-2
