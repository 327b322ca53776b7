"""`spatha.spmm` for PyTorch-ROCm: the operator the reference's end-to-end path
calls (end2end/spatha_mod/block_sparse/api/spatha.cu:41-65), served by
libspatha.so through its C ABI.  torch is used for device memory and the
current stream only."""
import ctypes
import weakref

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
        self._workspaces = {}          # stream -> zero-initialised scratch tensor of split runs
        self._finalizer = weakref.finalize(self, L.spatha_spmm_plan_destroy, handle)

    def kernel_name(self, N, out_layout=OUT_ROW_MAJOR, variant=0):
        name = _lib.lib().spatha_spmm_kernel_name(self._handle, N, out_layout, variant)
        return None if name is None else name.decode()

    def workspace_bytes(self, N, transposed_out=False, fused=False):
        """Bytes of scratch memory with which `run(..., split=True)` would split k-loops for N columns (0: never for this shape)."""
        return int(_lib.lib().spatha_spmm_workspace_bytes(self._handle, N, OUT_TRANSPOSED if transposed_out else OUT_ROW_MAJOR,
                                                          1 if fused else 0))

    def run(self, B, bias=None, transposed_out=False, variant=0, out=None, activation=None, split=False, workspace=None):
        """C = A B (or its transpose), fp16.  Without `activation`, a bias needs the transposed layout (the
        reference operator's contract).  With `activation` given ("none", "gelu", "gelu_tanh") the call goes through
        the fused entry point: out = act(fp16(A B) + bias) in either layout.
        split=True (automatic kernel choice only) lets the library split k-loops over workgroups where tiles alone leave CUs
        idle; the scratch memory it needs is `workspace` (a uint8 tensor on the GPU that was zero-filled once, e.g. by
        torch.zeros) or, if None, a buffer the plan keeps per stream."""
        _check_dev(B, torch.float16, "rhs")
        if B.dim() != 2 or B.shape[0] != self.cols:
            raise ValueError("rhs must be [%d, N], got %s" % (self.cols, tuple(B.shape)))
        N = B.shape[1]
        if bias is not None:
            _check_dev(bias, torch.float16, "bias")
            if bias.numel() != self.rows:
                raise ValueError("bias must have %d entries" % self.rows)
        if N % 8 != 0 and N > 0:
            # the library moves rows of B and C in 16-byte pieces: run on a copy with zero columns appended, cut the result back
            full = self.run(torch.nn.functional.pad(B, (0, 8 - N % 8)), bias, transposed_out, variant, None, activation, split,
                            workspace)
            cut = full[:N] if transposed_out else full[:, :N]
            if out is None:
                return cut.contiguous()
            _check_dev(out, torch.float16, "out")
            if tuple(out.shape) != tuple(cut.shape):
                raise ValueError("out must be %s" % (tuple(cut.shape),))
            out.copy_(cut)
            return out
        shape = (N, self.rows) if transposed_out else (self.rows, N)
        if out is None:
            out = torch.empty(shape, dtype=torch.float16, device=B.device)
        else:
            _check_dev(out, torch.float16, "out")
            if tuple(out.shape) != shape:
                raise ValueError("out must be %s" % (shape,))
        layout = OUT_TRANSPOSED if transposed_out else OUT_ROW_MAJOR
        if split:
            if variant != 0:
                raise ValueError("split=True goes with the automatic kernel choice (variant=0)")
            if activation is None and bias is not None and not transposed_out:
                raise RuntimeError("spatha_spmm_run: a bias needs the transposed layout (or an activation argument)")
            act = "none" if activation is None else activation
            if act not in _ACTIVATIONS:
                raise ValueError("unknown activation %r" % (activation,))
            fused = _ACTIVATIONS[act] != ACT_NONE or (bias is not None and not transposed_out)
            need = self.workspace_bytes(N, transposed_out, fused)
            if workspace is None and need:
                key = torch.cuda.current_stream(self.device).cuda_stream
                workspace = self._workspaces.get(key)
                if workspace is None or workspace.numel() < need:
                    workspace = self._workspaces[key] = torch.zeros(need, dtype=torch.uint8, device=B.device)
            ws_ptr = None if workspace is None else workspace.data_ptr()
            ws_len = 0 if workspace is None else workspace.numel() * workspace.element_size()
            with torch.cuda.device(self.device):
                _lib.check(_lib.lib().spatha_spmm_run_ws(self._handle, B.data_ptr(), N, None if bias is None else bias.data_ptr(),
                                                         out.data_ptr(), layout, _ACTIVATIONS[act], ws_ptr, ws_len,
                                                         _stream_ptr(self.device)), "spatha_spmm_run_ws")
            torch.autograd.graph.increment_version(out)
            return out
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

    def tune(self, B, out, bias=None, transposed_out=False, warmup=5, iters=30):
        """Times the automatic choice and every kernel id that accepts this shape; returns (best id, its ms, the automatic
        choice's ms, {id: ms}) with id 0 = the automatic choice (the best id is 0 when nothing beats it)."""
        L = _lib.lib()
        n = L.spatha_spmm_num_variants()
        best, best_ms, auto_ms = ctypes.c_int(), ctypes.c_float(), ctypes.c_float()
        per = (ctypes.c_float * n)()
        with torch.cuda.device(self.device):
            _lib.check(L.spatha_spmm_tune(self._handle, B.data_ptr(), B.shape[1], None if bias is None else bias.data_ptr(),
                                          out.data_ptr(), OUT_TRANSPOSED if transposed_out else OUT_ROW_MAJOR, warmup, iters,
                                          _stream_ptr(self.device), ctypes.byref(best), ctypes.byref(best_ms),
                                          ctypes.byref(auto_ms), per), "spatha_spmm_tune")
        torch.autograd.graph.increment_version(out)
        return best.value, best_ms.value, auto_ms.value, {i: per[i] for i in range(n) if per[i] >= 0}


def _extension():
    """The PyTorch C++ extension that holds the operator (csrc/spatha_torch.cpp, built in place by `python -m
    venom_amd.build`): `spmm` with the reference's signature, `spmm_fused`, and the cache of plans of the matrices they
    have seen.  There is no fallback: without it the operator raises."""
    try:
        from . import _spatha_torch
    except ImportError as e:
        raise RuntimeError("the PyTorch extension venom_amd/_spatha_torch.so is not built or does not load (%s): run "
                           "`python -m venom_amd.build`" % e)
    return _spatha_torch


def clear_plan_cache():
    _extension().clear_plan_cache()


def invalidate_plans(A_values):
    """Drops the operator's cached plans built from this values tensor; returns how many.  Needed only after the weights were
    changed in a way torch does not record (through `.data` or a raw pointer): in-place tensor operations bump the
    tensor's version, and the operator rebuilds (and drops the stale plan) by itself."""
    return int(_extension().invalidate_plans(A_values))


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


def add_layernorm(x, residual, weight, bias, eps, feature_major=False):
    """LayerNorm(x + residual) over the last dimension in one kernel (residual may be None): fp16 tensors on the GPU,
    x and residual contiguous and of the same shape, weight and bias of length x.shape[-1] (a multiple of 8, at most
    4096).  Same arithmetic as torch's addition followed by torch.nn.functional.layer_norm on fp16 tensors.
    feature_major=True returns (out, out_t): the kernel also writes the result as [hidden, tokens] (tokens a multiple
    of 8), which the next V:N:M projection takes as its right-hand side without a transposed copy."""
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
    if feature_major:
        tokens = x.numel() // hidden
        out_t = torch.empty((hidden, tokens), dtype=torch.float16, device=x.device)
        with torch.cuda.device(x.device):
            _lib.check(_lib.lib().spatha_add_layernorm_f16_t(x.data_ptr(), residual.data_ptr() if residual is not None else None,
                                                             weight.data_ptr(), bias.data_ptr(), float(eps), tokens, hidden,
                                                             out.data_ptr(), out_t.data_ptr(), _stream_ptr(x.device)),
                       "spatha_add_layernorm_f16_t")
        return out, out_t
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

    Same argument order and meaning as the reference operator (end2end/bert_pytorch.py:89-104), and like it a
    function of a PyTorch C++ extension (end2end/spatha_mod/block_sparse/api/spatha.cu:41-65).  vec_length is V and
    is honoured at run time; nnz and seed are accepted and unused, as there; mbrow/brow must be 32/4, the only layout
    the format defines.  Runs on torch's current stream."""
    return _extension().spmm(A_metadata, A_indices, A_values, rhs_matrix, bias, A_num_rows, A_num_cols, B_num_cols, vec_length,
                             n, m, nnz, seed, mbrow, brow)


def spmm_fused(A_metadata, A_indices, A_values, rhs_matrix, bias, A_num_rows, A_num_cols, vec_length, n, m,
               activation="none", transposed_out=False):
    """act((A_vnm @ rhs_matrix) + bias), fp16, as [A_num_rows, tokens] (default: ready to be the rhs of the next
    spmm without a transposed copy) or, with transposed_out, as [tokens, A_num_rows] like `spmm`."""
    if activation not in _ACTIVATIONS:
        raise ValueError("unknown activation %r" % (activation,))
    return _extension().spmm_fused(A_metadata, A_indices, A_values, rhs_matrix, bias, A_num_rows, A_num_cols, vec_length, n, m,
                                   _ACTIVATIONS[activation], transposed_out)
