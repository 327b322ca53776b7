"""GPT-2-large inference with every `Conv1D` projection stored in V:N:M and run through `spatha.spmm`.

Counterpart of the reference harness end2end/gpt2_pytorch.py (`SrnmSpmm` over
`transformers.pytorch_utils.Conv1D` :111-140, `linear_to_spmm` :159-173, timing :175-228).
`Conv1D` keeps its weight as [in_features, out_features] and computes x @ W + b, so the sparse
operand of the SpMM is W^T ([out, in]).  The reference encodes W as it lies and swaps the row / column
counts afterwards (:126-127), which times the right amount of work but does not compute the layer;
here the transposed weight is encoded, so the swapped model tracks the masked dense one.
The model is built from a local `GPT2Config` with random weights (no hub download): 36 layers,
width 1280, 20 heads, input 8 x 512 token ids below 100, as in the reference (:177-179).

    python -m venom_amd.gpt2 -m 8 -n 2 -v 64 [--layers 36] [--magnitude] [--repeats 30]
prints `algo,n,m,v,mean_ms,median_ms,std_ms,len` rows (first field 1, as the reference's GPT-2 script)."""
import argparse
import statistics
import timeit

import torch

from .bert import SrnmSpmm


class _AsLinear:
    """View of a Conv1D as the Linear it is equivalent to: weight [out, in], same bias."""

    def __init__(self, conv):
        self.weight = conv.weight.t().contiguous()
        self.bias = conv.bias


def conv1d_to_spmm(mod, n, m, v, magnitude=False):
    """Replaces, in place, every transformers Conv1D under `mod` (end2end/gpt2_pytorch.py:159-173)."""
    from transformers.pytorch_utils import Conv1D

    for name, child in list(mod.named_children()):
        if isinstance(child, Conv1D):
            setattr(mod, name, SrnmSpmm(_AsLinear(child), n, m, v, magnitude))
        elif not isinstance(child, SrnmSpmm):
            conv1d_to_spmm(child, n, m, v, magnitude)
    return mod


def build_gpt2_large(layers=36, seed=0, width=1280, heads=20):
    from transformers import GPT2Config, GPT2Model

    torch.manual_seed(seed)
    cfg = GPT2Config(n_embd=width, n_layer=layers, n_head=heads, n_positions=1024, vocab_size=50257)
    return GPT2Model(cfg).eval()


def report_time(name, data, n, m, v):
    ds = [d * 1000 for d in data]
    cfg = "%d,%d," % (n, m) if name == "n:m" else "0,0,"
    std = statistics.stdev(ds) if len(ds) > 1 else 0.0
    print("1," + cfg + "%d,%s,%s,%s,%d" % (v, statistics.mean(ds), statistics.median(ds), std, len(ds)), flush=True)
    return statistics.mean(ds)


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("-m", type=int, default=8)
    ap.add_argument("-n", type=int, default=2)
    ap.add_argument("-v", type=int, default=64)
    ap.add_argument("--layers", type=int, default=36)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--seq", type=int, default=512)
    ap.add_argument("--repeats", type=int, default=30)
    ap.add_argument("--magnitude", action="store_true", help="magnitude column selection instead of the fixed pattern")
    ap.add_argument("--fuse-ffn", action="store_true",
                    help="c_fc leaves its output (bias added in the kernel) feature-major for c_proj: no transposed copy of the "
                         "[tokens, 4*width] activation")
    ap.add_argument("--kernel-gelu", action="store_true", help="with --fuse-ffn: the activation in the kernel's write-out too")
    args = ap.parse_args(argv)
    torch.set_grad_enabled(False)
    dev = torch.device("cuda:0")
    dense_model = build_gpt2_large(args.layers).to(dev).half()
    sparse_model = conv1d_to_spmm(build_gpt2_large(args.layers).to(dev).half(), args.n, args.m, args.v, args.magnitude)
    if args.fuse_ffn:
        from .bert import fuse_feed_forward
        fuse_feed_forward(sparse_model, activation_in_kernel=args.kernel_gelu)
    ids = torch.randint(0, 100, (args.batch, args.seq), device=dev)

    def run(model):
        out = model(ids).last_hidden_state
        torch.cuda.synchronize()
        return out

    run(sparse_model)
    timeit.repeat(lambda: run(dense_model), repeat=5, number=1)
    t_dense = report_time("dense", timeit.repeat(lambda: run(dense_model), repeat=args.repeats, number=1), args.n, args.m, args.v)
    timeit.repeat(lambda: run(sparse_model), repeat=5, number=1)
    t_sparse = report_time("n:m", timeit.repeat(lambda: run(sparse_model), repeat=args.repeats, number=1), args.n, args.m, args.v)
    how = (" (fused feed-forward%s)" % (", activation in the kernel" if args.kernel_gelu else "")) if args.fuse_ffn else ""
    print("# dense %.2f ms, %d:%d:%d%s %.2f ms, speed-up %.2fx" % (t_dense, args.v, args.n, args.m, how, t_sparse, t_dense / t_sparse))


if __name__ == "__main__":
    main()
