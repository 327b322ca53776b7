"""BERT-large inference with every encoder Linear stored in V:N:M and run through `spatha.spmm`.

Counterpart of the reference harness end2end/bert_pytorch.py (`NMVectorSparsifier` :56-83,
`SrnmSpmm` :109-136, `linear_to_spmm` :155-167, timing :169-219).  Differences, on purpose:
the model is built from a local `BertConfig` with random weights (no hub download), only
`encoder.layer.*` Linears are swapped (the reference also swaps `pooler.dense`, whose 32-token
input is narrower than its kernel's tile), and where the STEN package is not installed its wrapper
is replaced by a two-method stand-in (only `wrapped_from_dense(...)` / `.wrapped_tensor` are used;
venom_amd/sten_registration.py holds it and the registration hooks for when STEN is there).

    python -m venom_amd.bert -m 8 -n 2 -v 64 [--layers 24] [--magnitude] [--repeats 30]
prints `algo,n,m,v,mean_ms,median_ms,std_ms,len` rows for the dense and the V:N:M model."""
import argparse
import statistics
import timeit

import torch

from . import spatha
from .grouped_nmv_tensor import SrNMTensor, nm_vector_mask_sparsify
from .sten_registration import SparseTensorWrapper, wrapper_class  # noqa: F401  (the stand-in keeps its old import path)


class NMVectorSparsifier:
    """magnitude=False: the reference harness's pattern (column-loc {0,1,2,3} in every group,
    mask [1,0,1,0,0,...]); magnitude=True: `nm_vector_mask_sparsify`."""

    def __init__(self, n, m, tileM, magnitude=False):
        self.n, self.m, self.tileM, self.magnitude = n, m, tileM, magnitude

    def __call__(self, tensor, grad_fmt=None):
        nrows, ncols = tensor.shape
        if self.magnitude:
            # model conversion: equal magnitudes (frequent in fp16 weights) go to the lower column, no history replay
            mask, columns = nm_vector_mask_sparsify(tensor, self.n, self.m, self.tileM, exact_ties=not tensor.is_cuda)
        else:
            columns = torch.arange(4, dtype=torch.int32).repeat(nrows // self.tileM, ncols // self.m)
            pat = torch.zeros(self.m, dtype=torch.int32)
            pat[0] = 1
            pat[2] = 1
            mask = pat.repeat(nrows, ncols // self.m)
        return wrapper_class().wrapped_from_dense(
            SrNMTensor(self.n, self.m, self.tileM, tensor, mask, columns, tensor.device), tensor, grad_fmt)


class SrnmSpmm(torch.nn.Module):
    """Drop-in for nn.Linear: y = x W^T + b with W in V:N:M."""

    def __init__(self, original, n, m, v, magnitude=False):
        super().__init__()
        self.n, self.m, self.v = n, m, v
        self.bias = original.bias
        w = NMVectorSparsifier(n, m, v, magnitude)(original.weight).wrapped_tensor
        self.values = torch.nn.Parameter(w.values, requires_grad=False)
        self.columns = w.columns
        self.metadata = w.metadata
        self.nrows_sp, self.ncols_sp, self.nnz = w.nrows, w.ncols, w.nnz

    # The query, key and value projections of a layer read the same activation: its transposed copy is
    # kept for the next call, keyed by address, shape and version counter of the input.  The input itself
    # is kept alive alongside, so that its address cannot be handed to another tensor while the entry exists.
    _last_rhs = (None, None, None)

    @classmethod
    def _transposed(cls, flat):
        if flat.stride(0) == 1 and flat.stride(1) == flat.shape[0]:
            return flat.T              # feature-major already (the output of a fused feed-forward layer): no copy
        key = (flat.data_ptr(), tuple(flat.shape), tuple(flat.stride()), flat._version, flat.device)
        if cls._last_rhs[0] == key:
            return cls._last_rhs[2]
        if flat.is_cuda and flat.dtype == torch.float16:
            rhs = spatha.transpose(flat.contiguous())
        else:
            rhs = flat.T.contiguous()
        cls._last_rhs = (key, flat, rhs)
        return rhs

    @classmethod
    def offer_transposed(cls, x, x_t):
        """A producer that has x[..., features] feature-major already (x_t[features, tokens]) leaves it for the layer that reads
        x next, in place of the transposed copy that layer would make."""
        flat = torch.flatten(x, start_dim=0, end_dim=-2)
        key = (flat.data_ptr(), tuple(flat.shape), tuple(flat.stride()), flat._version, flat.device)
        cls._last_rhs = (key, flat, x_t)

    _group = None          # set by merge_qkv: the projections this layer is computed together with
    _group_index = 0

    def forward(self, input):
        if self._group is not None:
            return self._group.output(self._group_index, self.nrows_sp, input)
        flat = torch.flatten(input, start_dim=0, end_dim=-2)          # [tokens, in]
        rhs = self._transposed(flat)                                  # [in, tokens], as the operator expects
        bias = self.bias if self.bias is not None else torch.zeros(self.nrows_sp, dtype=rhs.dtype, device=rhs.device)
        out = spatha.spmm(self.metadata, self.columns, self.values, rhs, bias, self.nrows_sp, self.ncols_sp,
                          rhs.shape[1], self.v, self.n, self.m, self.nnz, 0, 32, 4)   # [tokens, out]
        return out.reshape(*input.shape[:-1], -1)

    def forward_feature_major(self, input, activation="none"):
        """act(x W^T + b) as a [..., out] VIEW of a feature-major buffer [out, tokens]: bias and activation run in
        the kernel's write-out, and the next SrnmSpmm takes the buffer as its right-hand side without a copy."""
        flat = torch.flatten(input, start_dim=0, end_dim=-2)
        rhs = self._transposed(flat)
        out = spatha.spmm_fused(self.metadata, self.columns, self.values, rhs, self.bias, self.nrows_sp, self.ncols_sp,
                                self.v, self.n, self.m, activation=activation)              # [out, tokens]
        return out.T.reshape(*input.shape[:-1], -1)     # strides (.., 1, tokens): a view, nothing moves


class _MergedProjections:
    """Several SrnmSpmm layers that read the same activation (the query / key / value projections of an attention
    block) as ONE SpMM over the row-wise concatenation of their V:N:M matrices: the format is blocked by rows
    (values by 16, metadata by 32, column-loc by V), so the arrays simply concatenate.  The first member asked
    computes all of them; the others take their slice of the result while the activation is unchanged."""

    def __init__(self, layers):
        first = layers[0]
        assert all((l.ncols_sp, l.n, l.m, l.v) == (first.ncols_sp, first.n, first.m, first.v) for l in layers)
        self.v, self.n, self.m, self.cols = first.v, first.n, first.m, first.ncols_sp
        self.values = torch.cat([l.values.data for l in layers]).contiguous()
        self.metadata = torch.cat([l.metadata for l in layers]).contiguous()
        self.columns = torch.cat([l.columns for l in layers]).contiguous()
        zeros = [torch.zeros(l.nrows_sp, dtype=first.values.dtype, device=first.values.device) for l in layers]
        self.bias = torch.cat([l.bias.data if l.bias is not None else z for l, z in zip(layers, zeros)]).contiguous()
        self.starts, self.rows = [], 0
        for l in layers:
            self.starts.append(self.rows)
            self.rows += l.nrows_sp
        self._last = (None, None, None)          # (key, activation held alive, [tokens, rows] result)

    def output(self, index, nrows, input):
        flat = torch.flatten(input, start_dim=0, end_dim=-2)
        key = (flat.data_ptr(), tuple(flat.shape), tuple(flat.stride()), flat._version, flat.device)
        if self._last[0] != key:
            rhs = SrnmSpmm._transposed(flat)
            out = spatha.spmm(self.metadata, self.columns, self.values, rhs, self.bias, self.rows, self.cols, rhs.shape[1],
                              self.v, self.n, self.m, 0, 0, 32, 4)
            self._last = (key, flat, out)
        start = self.starts[index]
        return self._last[2][:, start:start + nrows].reshape(*input.shape[:-1], nrows)


def merge_qkv(model):
    """One SpMM instead of three for the query / key / value projections of every BertSelfAttention whose projections
    are SrnmSpmm layers (same numbers: every output row is computed exactly as before)."""
    from transformers.models.bert.modeling_bert import BertSelfAttention

    for mod in model.modules():
        if isinstance(mod, BertSelfAttention) and all(isinstance(getattr(mod, k), SrnmSpmm) for k in ("query", "key", "value")):
            layers = [mod.query, mod.key, mod.value]
            group = _MergedProjections(layers)
            for i, l in enumerate(layers):
                l._group, l._group_index = group, i
    return model


class FusedFeedForwardIn(torch.nn.Module):
    """Stands in for the Linear that opens a feed-forward block: one kernel computes x W^T + b (bias in the write-out)
    and leaves it feature-major, [out, tokens], which the block's second SrnmSpmm takes as its right-hand side as it
    lies, so the [tokens, 4*hidden] activation is never transposed.  The value returned is a [..., out] VIEW of that
    buffer; elementwise code between the two layers keeps its strides.
    activation: None (the caller applies its own), or "gelu" / "gelu_tanh" applied here, by torch's elementwise kernel
    (same bits as the unfused layers) or, with activation_in_kernel, in the SpMM's write-out (one pass less)."""

    def __init__(self, spmm_layer, activation=None, activation_in_kernel=False):
        super().__init__()
        self.dense = spmm_layer
        self.activation = activation
        self.activation_in_kernel = activation_in_kernel

    def forward(self, hidden_states):
        if self.activation is None:
            return self.dense.forward_feature_major(hidden_states, "none")
        if self.activation_in_kernel:
            return self.dense.forward_feature_major(hidden_states, self.activation)
        approx = "tanh" if self.activation != "gelu" else "none"
        return torch.nn.functional.gelu(self.dense.forward_feature_major(hidden_states, "none"), approximate=approx)


def fuse_feed_forward(model, activation_in_kernel=False):
    """Rewires, in place, every feed-forward block whose two projections are SrnmSpmm layers already: transformers'
    BertIntermediate (Linear + GELU) and GPT2MLP (c_fc, activation, c_proj).  Layers with V = 32, 96, ... keep the
    drop-in path (their kernels have no fused write-out)."""
    from transformers import activations as A
    from transformers.models.bert.modeling_bert import BertIntermediate
    from transformers.models.gpt2.modeling_gpt2 import GPT2MLP

    def kernel_name_of(fn):
        if isinstance(fn, A.GELUActivation) or fn is torch.nn.functional.gelu:
            return "gelu"
        if isinstance(fn, (A.NewGELUActivation, getattr(A, "PytorchGELUTanh", ()), getattr(A, "GELUTanh", ()))):
            return "gelu_tanh"
        return None

    for mod in model.modules():
        for name, child in list(mod.named_children()):
            if isinstance(child, BertIntermediate) and isinstance(child.dense, SrnmSpmm) and child.dense.v % 64 == 0:
                act = kernel_name_of(child.intermediate_act_fn)
                if act == "gelu":
                    setattr(mod, name, FusedFeedForwardIn(child.dense, act, activation_in_kernel))
            elif isinstance(child, GPT2MLP) and isinstance(child.c_fc, SrnmSpmm) and isinstance(child.c_proj, SrnmSpmm) \
                    and child.c_fc.v % 64 == 0:
                act = kernel_name_of(child.act)
                if activation_in_kernel and act is not None:
                    child.c_fc = FusedFeedForwardIn(child.c_fc, act, True)
                    child.act = torch.nn.Identity()
                else:
                    child.c_fc = FusedFeedForwardIn(child.c_fc, None)       # the block's own activation follows
    return model


class FusedProjectionNorm(torch.nn.Module):
    """Stands in for transformers' BertSelfOutput / BertOutput: the projection, then LayerNorm(projection + input) as ONE
    kernel (`spatha.add_layernorm`) instead of an addition and a normalisation.  Independent of the weight format: the
    projection may be an nn.Linear or an SrnmSpmm.  In training, or for tensors the kernel does not take, the stock
    sequence runs."""

    def __init__(self, mod, feature_major=False):
        super().__init__()
        self.dense, self.LayerNorm, self.dropout = mod.dense, mod.LayerNorm, mod.dropout
        # also write the result feature-major and hand that copy to the next SrnmSpmm (which would otherwise transpose it)
        self.feature_major = feature_major
        self.train(mod.training)

    def forward(self, hidden_states, input_tensor):
        h = self.dense(hidden_states)
        ln = self.LayerNorm
        if self.training or not h.is_cuda or h.dtype != torch.float16 or h.shape[-1] % 8 or h.shape[-1] > 4096 \
                or ln.weight is None or ln.bias is None:
            return ln(self.dropout(h) + input_tensor)
        h = h.contiguous()
        if self.feature_major and (h.numel() // h.shape[-1]) % 8 == 0:
            out, out_t = spatha.add_layernorm(h, input_tensor.contiguous(), ln.weight, ln.bias, ln.eps, feature_major=True)
            SrnmSpmm.offer_transposed(out, out_t)
            return out
        return spatha.add_layernorm(h, input_tensor.contiguous(), ln.weight, ln.bias, ln.eps)


def fuse_add_layernorm(model, feature_major=False):
    """Replaces, in place, every BertSelfOutput / BertOutput by FusedProjectionNorm (same parameters).  feature_major: for a
    model whose projections are SrnmSpmm layers - the kernel also writes the feature-major copy the next projection reads."""
    from transformers.models.bert.modeling_bert import BertOutput, BertSelfOutput

    for mod in model.modules():
        for name, child in list(mod.named_children()):
            if isinstance(child, (BertSelfOutput, BertOutput)):
                setattr(mod, name, FusedProjectionNorm(child, feature_major))
    return model


def linear_to_spmm(mod, n, m, v, magnitude=False, prefix="", only=("encoder.layer",)):
    """Replaces, in place, every nn.Linear whose qualified name contains one of `only`."""
    for name, child in list(mod.named_children()):
        full = prefix + "." + name if prefix else name
        if isinstance(child, torch.nn.Linear) and any(tag in full for tag in only):
            setattr(mod, name, SrnmSpmm(child, n, m, v, magnitude))
        elif not isinstance(child, SrnmSpmm):
            linear_to_spmm(child, n, m, v, magnitude, full, only)
    return mod


def report_time(name, data, number, n, m, v):
    ds = [d / number * 1000 for d in data]
    cfg = "%d,%d," % (n, m) if name == "n:m" else "0,0,"
    std = statistics.stdev(ds) if len(ds) > 1 else 0.0
    print("0," + cfg + "%d,%s,%s,%s,%d" % (v, statistics.mean(ds), statistics.median(ds), std, len(ds)), flush=True)
    return statistics.mean(ds)


def build_bert_large(layers=24, seed=0):
    from transformers import BertConfig, BertModel

    torch.manual_seed(seed)
    cfg = BertConfig(hidden_size=1024, num_hidden_layers=layers, num_attention_heads=16, intermediate_size=4096,
                     vocab_size=30522, max_position_embeddings=512)
    return BertModel(cfg).eval()


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("-m", type=int, default=8)
    ap.add_argument("-n", type=int, default=2)
    ap.add_argument("-v", type=int, default=64)
    ap.add_argument("--layers", type=int, default=24)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--seq", type=int, default=512)
    ap.add_argument("--repeats", type=int, default=30)
    ap.add_argument("--magnitude", action="store_true", help="magnitude column selection instead of the fixed pattern")
    ap.add_argument("--fuse-ffn", action="store_true",
                    help="first feed-forward layer of every block as one kernel (bias + GELU in the write-out, feature-major "
                         "result handed to the second layer without a transposed copy)")
    ap.add_argument("--merge-qkv", action="store_true", help="query, key and value projections of a block as one SpMM")
    ap.add_argument("--fuse-ln", action="store_true",
                    help="residual addition + LayerNorm after the attention-output and FFN-down projections as one kernel, "
                         "in BOTH models (the fusion does not depend on the weight format)")
    ap.add_argument("--ln-feature-major", action="store_true",
                    help="with --fuse-ln: the V:N:M model's residual + LayerNorm kernel also writes its result feature-major, the "
                         "layout the next projection reads (two of the three transposed copies per layer disappear)")
    ap.add_argument("--kernel-gelu", action="store_true",
                    help="with --fuse-ffn: GELU in the kernel's write-out too (default: torch's elementwise pass over the "
                         "feature-major buffer, which keeps the model's output bit-identical to the unfused layers)")
    args = ap.parse_args(argv)
    r = measure(args.n, args.m, args.v, layers=args.layers, batch=args.batch, seq=args.seq, repeats=args.repeats,
                magnitude=args.magnitude, fuse_ffn=args.fuse_ffn, merge=args.merge_qkv, fuse_ln=args.fuse_ln,
                kernel_gelu=args.kernel_gelu, report=True, ln_feature_major=args.ln_feature_major)
    print("# dense %.2f ms, %d:%d:%d%s %.2f ms, speed-up %.2fx" % (r["dense_ms"], args.v, args.n, args.m,
                                                                    ((" (fused feed-forward%s)" % (", activation in the kernel" if args.kernel_gelu else "")) if args.fuse_ffn else "")
                                                                    + (" (merged q/k/v)" if args.merge_qkv else "")
                                                                    + (" (fused add + LayerNorm in both%s)" % (", feature-major copy for the next projection" if args.ln_feature_major else "") if args.fuse_ln else ""), r["vnm_ms"],
                                                                    r["speedup"]))


def measure(n=2, m=8, v=64, layers=24, batch=32, seq=512, repeats=30, warmups=5, magnitude=False, fuse_ffn=False, merge=False,
            fuse_ln=False, kernel_gelu=False, report=False, ln_feature_major=False):
    """Times the dense fp16 encoder and the same encoder with its Linears in V:N:M on cuda:0 (the reference's procedure,
    end2end/bert_pytorch.py:211-219: warm-ups, then `repeats` forward passes timed one by one, each ended by a device
    synchronisation); returns mean and median milliseconds of both and their ratio."""
    import copy

    prev_grad = torch.is_grad_enabled()
    torch.set_grad_enabled(False)
    try:
        dev = torch.device("cuda:0")
        base = build_bert_large(layers)
        dense_model = copy.deepcopy(base).to(dev).half()
        sparse_model = linear_to_spmm(base.to(dev).half(), n, m, v, magnitude)
        if fuse_ffn:
            fuse_feed_forward(sparse_model, activation_in_kernel=kernel_gelu)
        if merge:
            merge_qkv(sparse_model)
        if fuse_ln:
            fuse_add_layernorm(dense_model)
            fuse_add_layernorm(sparse_model, feature_major=ln_feature_major)
        ids = torch.randint(0, 30522, (batch, seq), device=dev)

        def run(model):
            out = model(ids).last_hidden_state
            torch.cuda.synchronize()
            return out

        run(sparse_model)
        timeit.repeat(lambda: run(dense_model), repeat=warmups, number=1)
        d = [t * 1e3 for t in timeit.repeat(lambda: run(dense_model), repeat=repeats, number=1)]
        timeit.repeat(lambda: run(sparse_model), repeat=warmups, number=1)
        s = [t * 1e3 for t in timeit.repeat(lambda: run(sparse_model), repeat=repeats, number=1)]
        if report:
            report_time("dense", [t / 1e3 for t in d], 1, n, m, v)
            report_time("n:m", [t / 1e3 for t in s], 1, n, m, v)
        spatha.clear_plan_cache()
        return {"dense_ms": round(statistics.mean(d), 3), "vnm_ms": round(statistics.mean(s), 3),
                "dense_median_ms": round(statistics.median(d), 3), "vnm_median_ms": round(statistics.median(s), 3),
                "speedup": round(statistics.mean(d) / statistics.mean(s), 3), "repeats": repeats,
                "format": "%d:%d:%d" % (v, n, m), "layers": layers, "tokens": batch * seq}
    finally:
        torch.set_grad_enabled(prev_grad)


if __name__ == "__main__":
    main()
