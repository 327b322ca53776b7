"""Registration of the V:N:M format with STEN (the sparse-tensor framework the reference's end-to-end path is written
against: end2end/tests.ipynb cells 14 and 24, `sten.SparseTensorWrapper` in end2end/bert_pytorch.py:77-83).

STEN is a separate package.  Where it can be imported, `register()` hooks the two pieces of the reference's notebook up to
this library:

  * the sparsifier implementation  NMVectorSparsifier: torch.Tensor -> SrNMTensor  (magnitude selection through
    `nm_vector_mask_sparsify`, wrapped with `sten.SparseTensorWrapper.wrapped_from_dense`);
  * the forward implementation of `torch.mm(SrNMTensor, torch.Tensor)` through `spatha.spmm` (no bias, result
    [A_num_rows, B_num_cols] like `torch.mm`).

Where it cannot, `register()` raises ImportError and `wrapper_class()` hands out the two-method stand-in the harnesses need
(`wrapped_from_dense(...)`, `.wrapped_tensor`).  `register(sten_module)` takes the module as an argument so that the hooks can
be exercised against any object with STEN's registration interface."""
import torch

from . import spatha
from .grouped_nmv_tensor import SrNMTensor, nm_vector_mask_sparsify


class SparseTensorWrapper:
    """The part of sten.SparseTensorWrapper the harnesses use."""

    def __init__(self, wrapped_tensor, dense, grad_fmt=None):
        self.wrapped_tensor = wrapped_tensor
        self.dense_shape = tuple(dense.shape)
        self.grad_fmt = grad_fmt

    @staticmethod
    def wrapped_from_dense(wrapped_tensor, dense, grad_fmt=None):
        return SparseTensorWrapper(wrapped_tensor, dense, grad_fmt)


def sten_module():
    """The STEN package, or None where it is not installed."""
    try:
        import sten
    except ImportError:
        return None
    return sten


def wrapper_class():
    """sten.SparseTensorWrapper where STEN is installed, the stand-in otherwise."""
    sten = sten_module()
    return SparseTensorWrapper if sten is None else sten.SparseTensorWrapper


def srnm_mm(lhs, rhs):
    """torch.mm(A, rhs) with A an SrNMTensor: [A.nrows, rhs.shape[1]] in fp16 on A's device."""
    dev = lhs.values.device
    rhs16 = rhs.to(device=dev, dtype=torch.float16).contiguous()
    out = spatha.spmm_fused(lhs.metadata, lhs.columns, lhs.values, rhs16, None, lhs.nrows, lhs.ncols, lhs.tileM, lhs.n, lhs.m)
    return out


def register(sten=None, sparsifier_class=None):
    """Registers the sparsifier implementation and the torch.mm forward implementation with STEN.  `sparsifier_class` is the
    class whose instances carry n, m and tileM (default: the harness's NMVectorSparsifier).  Returns the two registered
    functions."""
    if sten is None:
        sten = sten_module()
        if sten is None:
            raise ImportError("STEN is not installed: `import sten` fails")
    if sparsifier_class is None:
        from .bert import NMVectorSparsifier as sparsifier_class

    @sten.register_sparsifier_implementation(sparsifier=sparsifier_class, inp=torch.Tensor, out=SrNMTensor)
    def torch_tensor_to_srnm(sparsifier, tensor, grad_fmt=None):
        masks, columns = nm_vector_mask_sparsify(tensor, sparsifier.n, sparsifier.m, sparsifier.tileM)
        return sten.SparseTensorWrapper.wrapped_from_dense(
            SrNMTensor(sparsifier.n, sparsifier.m, sparsifier.tileM, tensor, masks, columns, tensor.device), tensor, grad_fmt)

    @sten.register_fwd_op_impl(operator=torch.mm, inp=(SrNMTensor, torch.Tensor), out=[(sten.KeepAll, torch.Tensor)])
    def srnm_mm_fwd_impl(ctx, inputs, output_sparsifiers):
        lhs, rhs = inputs
        ctx.save_for_backward(lhs, rhs)
        return srnm_mm(lhs.wrapped_tensor, rhs)

    return torch_tensor_to_srnm, srnm_mm_fwd_impl
