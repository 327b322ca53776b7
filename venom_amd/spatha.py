"""`spatha.spmm` for PyTorch-ROCm: the operator the reference's end-to-end path
calls (end2end/spatha_mod/block_sparse/api/spatha.cu:41-65), served by
libspatha.so through its C ABI.  torch is used for device memory and the
current stream only."""
import ctypes
import weakref
from collections import OrderedDict

import torch

from . import _lib

OUT_ROW_MAJOR = 0
OUT_TRANSPOSED = 1
ACT_NONE, ACT_GELU, ACT_GELU_TANH = 0, 1, 2
_ACTIVATIONS = {None: ACT_NONE, "none": ACT_NONE, "gelu": ACT_GELU, "gelu_tanh": ACT_GELU_TANH, "gelu_new": ACT_GELU_TANH,
                "gelu_pytorch_tanh": ACT_GELU_TANH}


def num_variants():
    """Kernel variants are numbered 1 .. num_variants() - 1; 0 selects automatically."""
    return int(_lib.lib().spatha_spmm_num_variants())


def _stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _check_dev(t, dtype, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError("%s must be a tensor on the GPU" % name)
    if t.dtype != dtype:
        raise TypeError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)


class SpmmPlan:
    """Owns the library's plan (the copies of A laid out for the sparse matrix
    instructions) for one V:N:M matrix."""

    def __init__(self, values, metadata, columns, rows, cols, n, m, v):
        _check_dev(values, torch.float16, "values")
        _check_dev(metadata, torch.int32, "metadata")
        _check_dev(columns, torch.int32, "columns")
        g = _lib.Geometry()
        L = _lib.lib()
        _lib.check(L.spatha_vnm_geometry_init(rows, cols, n, m, v, ctypes.byref(g)), "spatha_vnm_geometry_init")
        if values.numel() != g.n_values or metadata.numel() != g.n_metadata or columns.numel() != g.n_columns:
            raise ValueError("values/metadata/columns sizes (%d, %d, %d) do not match the V:N:M geometry (%d, %d, %d)" % (
                values.numel(), metadata.numel(), columns.numel(), g.n_values, g.n_metadata, g.n_columns))
        self.rows, self.cols, self.n, self.m, self.v, self.ksp = rows, cols, n, m, v, g.ksp
        self.device = values.device
        handle = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            _lib.check(L.spatha_spmm_plan_create(rows, cols, n, m, v, values.data_ptr(), metadata.data_ptr(),
                                                 columns.data_ptr(), _stream_ptr(self.device), ctypes.byref(handle)),
                       "spatha_spmm_plan_create")
        self._handle = handle
        self._finalizer = weakref.finalize(self, L.spatha_spmm_plan_destroy, handle)

    def kernel_name(self, N, out_layout=OUT_ROW_MAJOR, variant=0):
        name = _lib.lib().spatha_spmm_kernel_name(self._handle, N, out_layout, variant)
        return None if name is None else name.decode()

    def run(self, B, bias=None, transposed_out=False, variant=0, out=None, activation=None):
        """C = A B (or its transpose), fp16.  Without `activation`, a bias needs the transposed layout (the
        reference operator's contract).  With `activation` given ("none", "gelu", "gelu_tanh") the call goes through
        the fused entry point: out = act(fp16(A B) + bias) in either layout."""
        _check_dev(B, torch.float16, "rhs")
        if B.dim() != 2 or B.shape[0] != self.cols:
            raise ValueError("rhs must be [%d, N], got %s" % (self.cols, tuple(B.shape)))
        N = B.shape[1]
        if bias is not None:
            _check_dev(bias, torch.float16, "bias")
            if bias.numel() != self.rows:
                raise ValueError("bias must have %d entries" % self.rows)
        shape = (N, self.rows) if transposed_out else (self.rows, N)
        if out is None:
            out = torch.empty(shape, dtype=torch.float16, device=B.device)
        else:
            _check_dev(out, torch.float16, "out")
            if tuple(out.shape) != shape:
                raise ValueError("out must be %s" % (shape,))
        layout = OUT_TRANSPOSED if transposed_out else OUT_ROW_MAJOR
        with torch.cuda.device(self.device):
            if activation is None:
                _lib.check(_lib.lib().spatha_spmm_run(self._handle, B.data_ptr(), N,
                                                      None if bias is None else bias.data_ptr(), out.data_ptr(), layout,
                                                      variant, _stream_ptr(self.device)), "spatha_spmm_run")
            else:
                if activation not in _ACTIVATIONS:
                    raise ValueError("unknown activation %r" % (activation,))
                _lib.check(_lib.lib().spatha_spmm_run_fused(self._handle, B.data_ptr(), N,
                                                            None if bias is None else bias.data_ptr(), out.data_ptr(),
                                                            layout, _ACTIVATIONS[activation], variant,
                                                            _stream_ptr(self.device)), "spatha_spmm_run_fused")
        # the kernel wrote through a raw pointer: tell torch, so that caches keyed on the tensor's version see the change
        torch.autograd.graph.increment_version(out)
        return out

    def time(self, B, out, bias=None, transposed_out=False, variant=0, warmup=10, iters=100):
        """Mean milliseconds per launch, HIP events on the current stream."""
        ms = ctypes.c_float()
        with torch.cuda.device(self.device):
            _lib.check(_lib.lib().spatha_spmm_time(self._handle, B.data_ptr(), B.shape[1],
                                                   None if bias is None else bias.data_ptr(), out.data_ptr(),
                                                   OUT_TRANSPOSED if transposed_out else OUT_ROW_MAJOR, variant,
                                                   warmup, iters, _stream_ptr(self.device), ctypes.byref(ms)),
                       "spatha_spmm_time")
        return ms.value


# plans of matrices already seen by spmm(), keyed by the identity and version of
# the three tensors; the entry keeps the tensors alive so that an address cannot
# be recycled under a stale plan
_PLAN_CACHE = OrderedDict()
_PLAN_CACHE_MAX = 1024


def _plan_for(values, metadata, columns, rows, cols, n, m, v):
    key = (values.data_ptr(), metadata.data_ptr(), columns.data_ptr(), values._version, metadata._version,
           columns._version, rows, cols, n, m, v)
    hit = _PLAN_CACHE.get(key)
    if hit is not None:
        _PLAN_CACHE.move_to_end(key)
        return hit[0]
    plan = SpmmPlan(values, metadata, columns, rows, cols, n, m, v)
    _PLAN_CACHE[key] = (plan, values, metadata, columns)
    while len(_PLAN_CACHE) > _PLAN_CACHE_MAX:
        _PLAN_CACHE.popitem(last=False)
    return plan


def clear_plan_cache():
    _PLAN_CACHE.clear()


def transpose(x):
    """x[rows, cols] fp16, contiguous -> a new contiguous [cols, rows] tensor (what `x.T.contiguous()` returns),
    through the library's tiled kernel on torch's current stream."""
    _check_dev(x, torch.float16, "x")
    if x.dim() != 2:
        raise ValueError("transpose expects a matrix")
    out = torch.empty((x.shape[1], x.shape[0]), dtype=torch.float16, device=x.device)
    if x.numel():
        with torch.cuda.device(x.device):
            _lib.check(_lib.lib().spatha_transpose_f16(x.data_ptr(), x.shape[0], x.shape[1], out.data_ptr(),
                                                       _stream_ptr(x.device)), "spatha_transpose_f16")
    return out


def add_layernorm(x, residual, weight, bias, eps):
    """LayerNorm(x + residual) over the last dimension in one kernel (residual may be None): fp16 tensors on the GPU,
    x and residual contiguous and of the same shape, weight and bias of length x.shape[-1] (a multiple of 8, at most
    4096).  Same arithmetic as torch's addition followed by torch.nn.functional.layer_norm on fp16 tensors."""
    _check_dev(x, torch.float16, "x")
    hidden = x.shape[-1]
    if residual is not None:
        _check_dev(residual, torch.float16, "residual")
        if residual.shape != x.shape:
            raise ValueError("residual must have the shape of x")
    _check_dev(weight, torch.float16, "weight")
    _check_dev(bias, torch.float16, "bias")
    if weight.numel() != hidden or bias.numel() != hidden:
        raise ValueError("weight and bias must have x.shape[-1] elements")
    out = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device(x.device):
            _lib.check(_lib.lib().spatha_add_layernorm_f16(x.data_ptr(), residual.data_ptr() if residual is not None else None,
                                                           weight.data_ptr(), bias.data_ptr(), float(eps),
                                                           x.numel() // hidden, hidden, out.data_ptr(), _stream_ptr(x.device)),
                       "spatha_add_layernorm_f16")
    return out


def spmm(A_metadata, A_indices, A_values, rhs_matrix, bias, A_num_rows, A_num_cols, B_num_cols, vec_length, n, m,
         nnz=0, seed=0, mbrow=32, brow=4):
    """out[B_num_cols, A_num_rows] = (A_vnm @ rhs_matrix).T + bias, fp16.

    Same argument order and meaning as the reference operator
    (end2end/bert_pytorch.py:89-104).  vec_length is V and is honoured at run
    time; nnz and seed are accepted and unused, as there; mbrow/brow must be
    32/4, the only layout the format defines.  Runs on torch's current stream."""
    if mbrow != 32 or brow != 4:
        raise ValueError("only mbrow=32, brow=4 is defined for the V:N:M layout")
    if rhs_matrix.shape[1] != B_num_cols:
        raise ValueError("B_num_cols does not match rhs_matrix")
    plan = _plan_for(A_values.detach(), A_metadata, A_indices, A_num_rows, A_num_cols, n, m, vec_length)
    return plan.run(rhs_matrix, bias=bias, transposed_out=True)


def spmm_fused(A_metadata, A_indices, A_values, rhs_matrix, bias, A_num_rows, A_num_cols, vec_length, n, m,
               activation="none", transposed_out=False):
    """act((A_vnm @ rhs_matrix) + bias), fp16, as [A_num_rows, tokens] (default: ready to be the rhs of the next
    spmm without a transposed copy) or, with transposed_out, as [tokens, A_num_rows] like `spmm`."""
    plan = _plan_for(A_values.detach(), A_metadata, A_indices, A_num_rows, A_num_cols, n, m, vec_length)
    return plan.run(rhs_matrix, bias=bias, transposed_out=transposed_out, activation=activation)
