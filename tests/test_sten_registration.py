"""The STEN hooks (venom_amd/sten_registration.py) against a stand-in for the package's registration interface: STEN itself
is not installed here (its submodule is empty in the reference), so what is checked is that the hooks register what the
reference's notebook registers (end2end/tests.ipynb cells 14 and 24) and that the registered functions compute the right
thing; how STEN dispatches to them is STEN's business and is not covered."""
import types

import numpy as np
import pytest
import torch

from venom_amd import sten_registration as R
from venom_amd.grouped_nmv_tensor import SrNMTensor


class _Sparsifier:
    def __init__(self, n, m, tileM):
        self.n, self.m, self.tileM = n, m, tileM


def _fake_sten():
    calls = {}

    def register_sparsifier_implementation(sparsifier, inp, out):
        def deco(fn):
            calls["sparsifier"] = (sparsifier, inp, out, fn)
            return fn
        return deco

    def register_fwd_op_impl(operator, inp, out):
        def deco(fn):
            calls["fwd"] = (operator, inp, out, fn)
            return fn
        return deco

    mod = types.SimpleNamespace(register_sparsifier_implementation=register_sparsifier_implementation,
                                register_fwd_op_impl=register_fwd_op_impl, SparseTensorWrapper=R.SparseTensorWrapper,
                                KeepAll=type("KeepAll", (), {}))
    return mod, calls


def test_without_sten_the_harness_gets_the_stand_in():
    if R.sten_module() is not None:
        pytest.skip("STEN is installed")
    assert R.wrapper_class() is R.SparseTensorWrapper
    with pytest.raises(ImportError):
        R.register()


def test_hooks_register_what_the_notebook_registers():
    mod, calls = _fake_sten()
    to_srnm, mm_impl = R.register(mod, sparsifier_class=_Sparsifier)
    sparsifier, inp, out, fn = calls["sparsifier"]
    assert (sparsifier, inp, out) == (_Sparsifier, torch.Tensor, SrNMTensor) and fn is to_srnm
    operator, inp, out, fn = calls["fwd"]
    assert operator is torch.mm and inp == (SrNMTensor, torch.Tensor) and out == [(mod.KeepAll, torch.Tensor)] and fn is mm_impl
    # the sparsifier implementation: magnitude selection, wrapped; decoding gives the masked weights
    torch.manual_seed(0)
    w = torch.randn(128, 96)
    wrapped = to_srnm(_Sparsifier(2, 8, 64), w)
    t = wrapped.wrapped_tensor
    assert isinstance(t, SrNMTensor) and (t.n, t.m, t.tileM, t.nrows, t.ncols) == (2, 8, 64, 128, 96)
    dense = t.to_dense().float()
    kept = dense != 0
    assert kept.sum().item() == 128 * 96 // 4
    assert torch.equal(dense[kept], w.half().float()[kept])
    # per row and group of 8 columns the two largest magnitudes among the block's four columns survive: at least the kept
    # entries are never smaller than every dropped one of their group
    g = w.abs().reshape(128, 12, 8)
    k = kept.reshape(128, 12, 8)
    assert bool((k.sum(-1) == 2).all())


@pytest.mark.gpu
def test_registered_mm_runs_the_sparse_kernel(gpu):
    mod, calls = _fake_sten()
    to_srnm, mm_impl = R.register(mod, sparsifier_class=_Sparsifier)
    torch.manual_seed(1)
    w = torch.randint(-4, 5, (256, 320)).float().to(gpu)
    rhs = torch.randint(-3, 4, (320, 72)).float().to(gpu)
    wrapped = to_srnm(_Sparsifier(2, 10, 64), w)
    saved = []
    ctx = types.SimpleNamespace(save_for_backward=lambda *a: saved.append(a))
    out = mm_impl(ctx, (wrapped, rhs), None)
    assert len(saved) == 1 and saved[0][0] is wrapped
    want = wrapped.wrapped_tensor.to_dense().float() @ rhs
    assert out.shape == (256, 72) and out.dtype == torch.float16
    assert np.array_equal(out.float().cpu().numpy(), want.cpu().numpy())
