"""spatha_spmm_run_noalloc (derived copies of A in the library's fixed device array, no allocation) against
spatha_spmm_plan_create + spatha_spmm_run, through the C ABI, bit for bit: two calls in a row, the second with a smaller
matrix, so that what the first call left in the array must not show."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from venom_amd import _lib
from venom_amd import format as F

pytestmark = pytest.mark.gpu


def _dev(a, gpu):
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(np.ascontiguousarray(a)).to(gpu)


def _both(gpu, rows, cols, N, m, v, transposed, seed):
    L = _lib.lib()
    vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=seed, integer_values=True)
    rng = np.random.default_rng(seed + 1)
    B = _dev(rng.integers(-4, 5, size=(cols, N)).astype(np.float16), gpu)
    bias = _dev(rng.integers(-3, 4, size=rows).astype(np.float16), gpu) if transposed else None
    dv, dm, dc = _dev(vals, gpu), _dev(meta, gpu), _dev(columns, gpu)
    shape = (N, rows) if transposed else (rows, N)
    stream = ctypes.c_void_p(torch.cuda.current_stream(gpu).cuda_stream)
    bias_ptr = None if bias is None else bias.data_ptr()
    layout = 1 if transposed else 0
    # a poisoned output buffer: every element must be written
    got = torch.full(shape, float("nan"), dtype=torch.float16, device=gpu)
    st = L.spatha_spmm_run_noalloc(rows, cols, 2, m, v, dv.data_ptr(), dm.data_ptr(), dc.data_ptr(), B.data_ptr(), N, bias_ptr,
                                   got.data_ptr(), layout, stream)
    assert st == 0, L.spatha_status_string(st)
    torch.cuda.synchronize()
    handle = ctypes.c_void_p()
    _lib.check(L.spatha_spmm_plan_create(rows, cols, 2, m, v, dv.data_ptr(), dm.data_ptr(), dc.data_ptr(), stream,
                                         ctypes.byref(handle)), "plan_create")
    want = torch.empty(shape, dtype=torch.float16, device=gpu)
    _lib.check(L.spatha_spmm_run(handle, B.data_ptr(), N, bias_ptr, want.data_ptr(), layout, 0, stream), "run")
    torch.cuda.synchronize()
    _lib.check(L.spatha_spmm_plan_destroy(handle), "plan_destroy")
    return got, want


@pytest.mark.parametrize("transposed", [False, True])
def test_noalloc_entry_point_equals_the_plan_path_twice_in_a_row(gpu, transposed):
    print("no-alloc entry point, transposed", transposed, flush=True)
    # first a matrix that fills most of the array (4096 x 1024 at 2:8 on the unified kernel for N = 4096) ...
    got, want = _both(gpu, 4096, 1024, 4096, 8, 64, transposed, seed=11)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # ... then a smaller one with another format (m = 16, V = 128, K tail, ragged N): stale contents must not matter
    got, want = _both(gpu, 512, 650, 136, 16, 128, transposed, seed=12)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # and a half-tile format (V = 32) after it
    got, want = _both(gpu, 256, 200, 72, 8, 32, transposed, seed=13)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_noalloc_entry_point_rejects_what_does_not_fit(gpu):
    L = _lib.lib()
    one = torch.zeros(16, dtype=torch.float16, device=gpu)
    # 16384 x 4096 at 2:8: 37.7 MB of packed operands
    st = L.spatha_spmm_run_noalloc(16384, 4096, 2, 8, 64, one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(), 64, None,
                                   one.data_ptr(), 0, None)
    assert st == 6 and b"capacity" in L.spatha_status_string(st)
    assert L.spatha_spmm_run_noalloc(100, 128, 2, 8, 64, one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(), 64, None,
                                     one.data_ptr(), 0, None) == 2           # rows % V
    assert L.spatha_spmm_run_noalloc(128, 128, 2, 8, 64, None, one.data_ptr(), one.data_ptr(), one.data_ptr(), 64, None,
                                     one.data_ptr(), 0, None) == 1


def test_noalloc_entry_point_refuses_before_it_launches(gpu):
    """A call that is going to be refused (N % 8, a bias with the row-major layout, a misaligned B) returns its status
    before any kernel is launched, so it cannot have rewritten the array under a valid call: after such calls a valid
    call still gives the right result, and the refused calls left their output buffers alone."""
    L = _lib.lib()
    rows, cols, N, m, v = 256, 512, 72, 8, 64
    vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=31, integer_values=True)
    B = np.random.default_rng(31).integers(-4, 5, size=(cols, N)).astype(np.float16)
    dv, dm, dc, dB = _dev(vals, gpu), _dev(meta, gpu), _dev(columns, gpu), _dev(B, gpu)
    out = torch.full((rows, N), 7.0, dtype=torch.float16, device=gpu)
    args = (rows, cols, 2, m, v, dv.data_ptr(), dm.data_ptr(), dc.data_ptr())
    assert L.spatha_spmm_run_noalloc(*args, dB.data_ptr(), 12, None, out.data_ptr(), 0, None) == 2         # N % 8
    assert L.spatha_spmm_run_noalloc(*args, dB.data_ptr(), N, dv.data_ptr(), out.data_ptr(), 0, None) == 1  # bias, row-major
    assert L.spatha_spmm_run_noalloc(*args, dB.data_ptr() + 2, N, None, out.data_ptr(), 0, None) == 1       # B not 16-byte aligned
    assert L.spatha_spmm_run_noalloc(*args, dB.data_ptr(), N, None, out.data_ptr(), 5, None) == 1           # layout
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())
    assert L.spatha_spmm_run_noalloc(*args, dB.data_ptr(), N, None, out.data_ptr(), 0, None) == 0
    torch.cuda.synchronize()
    want = oracle.spmm(vals, meta, columns, rows, cols, 2, m, v, B)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_noalloc_entry_point_recorded_into_a_graph(gpu):
    """After one eager call on the device (the first call looks up the array's address and sets kernel attributes, which a
    capture cannot hold), a call is recorded into a graph: three replays with new contents of A's values and of B,
    eager work and synchronisations between them, each equal to the oracle."""
    L = _lib.lib()
    rows, cols, N, m, v = 512, 650, 136, 16, 128
    vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=41, integer_values=True)
    rng = np.random.default_rng(41)
    B = rng.integers(-4, 5, size=(cols, N)).astype(np.float16)
    dv, dm, dc, dB = _dev(vals, gpu), _dev(meta, gpu), _dev(columns, gpu), _dev(B, gpu)
    out = torch.empty((rows, N), dtype=torch.float16, device=gpu)

    def call():
        stream = ctypes.c_void_p(torch.cuda.current_stream(gpu).cuda_stream)
        st = L.spatha_spmm_run_noalloc(rows, cols, 2, m, v, dv.data_ptr(), dm.data_ptr(), dc.data_ptr(), dB.data_ptr(), N, None,
                                       out.data_ptr(), 0, stream)
        assert st == 0, L.spatha_status_string(st)

    call()                                  # the warm-up call, outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        B = rng.integers(-4, 5, size=(cols, N)).astype(np.float16)
        vals2 = (vals * (rep + 1)).astype(np.float16) if rep < 2 else vals
        dB.copy_(_dev(B, gpu))
        dv.copy_(_dev(vals2, gpu))
        out.zero_()
        # another matrix through the same array between the replays: the replay has to rewrite everything it reads
        other = _both(gpu, 256, 200, 72, 8, 32, False, seed=50 + rep)
        assert torch.equal(other[0].view(torch.int16), other[1].view(torch.int16))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = oracle.spmm(vals2, meta, columns, rows, cols, 2, m, v, B)
        assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16)), rep
