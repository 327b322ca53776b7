"""One GPT-3-175B-sized transformer block (width 12288, 96 heads) with its `Conv1D` projections in V:N:M.

Counterpart of the reference harness end2end/gpt3_pytorch.py (:177-228): a single `GPT2Block` built from a
local `GPT2Config` with random weights, input 1 x 4096 x 12288 fp16.  Only the block is constructed (the
reference builds the whole language model and keeps `transformer.h[0]`).  The projections are replaced as in
`venom_amd.gpt2` (the transposed `Conv1D` weight is what gets encoded).

    python -m venom_amd.gpt3 -m 8 -n 2 -v 64 [--tokens 4096] [--repeats 30]
prints `algo,n,m,v,mean_ms,median_ms,std_ms,len` rows (first field 2, as the reference's GPT-3 script)."""
import argparse
import statistics
import timeit

import torch

from .gpt2 import conv1d_to_spmm


def build_gpt3_block(width=12288, heads=96, positions=4096, seed=0):
    from transformers import GPT2Config
    from transformers.models.gpt2.modeling_gpt2 import GPT2Block

    torch.manual_seed(seed)
    cfg = GPT2Config(vocab_size=50257, n_positions=positions, n_embd=width, n_layer=1, n_head=heads,
                     activation_function="gelu", resid_pdrop=0.1, embd_pdrop=0.1, attn_pdrop=0.1,
                     layer_norm_epsilon=1e-5, initializer_range=0.02)
    cfg._attn_implementation = "sdpa"
    return GPT2Block(cfg, layer_idx=0).eval()


def report_time(name, data, n, m, v):
    ds = [d * 1000 for d in data]
    cfg = "%d,%d," % (n, m) if name == "n:m" else "0,0,"
    std = statistics.stdev(ds) if len(ds) > 1 else 0.0
    print("2," + cfg + "%d,%s,%s,%s,%d" % (v, statistics.mean(ds), statistics.median(ds), std, len(ds)), flush=True)
    return statistics.mean(ds)


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("-m", type=int, default=8)
    ap.add_argument("-n", type=int, default=2)
    ap.add_argument("-v", type=int, default=64)
    ap.add_argument("--width", type=int, default=12288)
    ap.add_argument("--heads", type=int, default=96)
    ap.add_argument("--tokens", type=int, default=4096)
    ap.add_argument("--repeats", type=int, default=30)
    ap.add_argument("--magnitude", action="store_true")
    ap.add_argument("--fuse-ffn", action="store_true", help="c_fc leaves its output feature-major for c_proj (bias in the kernel)")
    ap.add_argument("--kernel-gelu", action="store_true", help="with --fuse-ffn: the activation in the kernel's write-out too")
    args = ap.parse_args(argv)
    torch.set_grad_enabled(False)
    dev = torch.device("cuda:0")
    dense_block = build_gpt3_block(args.width, args.heads, args.tokens).half().to(dev)
    sparse_block = conv1d_to_spmm(build_gpt3_block(args.width, args.heads, args.tokens).half().to(dev), args.n, args.m, args.v,
                                  args.magnitude)
    if args.fuse_ffn:
        from .bert import fuse_feed_forward
        fuse_feed_forward(sparse_block, activation_in_kernel=args.kernel_gelu)
    x = torch.rand((1, args.tokens, args.width), device=dev).half()

    def run(block):
        out = block(x)
        out = out[0] if isinstance(out, tuple) else out
        torch.cuda.synchronize()
        return out

    run(sparse_block)
    timeit.repeat(lambda: run(dense_block), repeat=5, number=1)
    t_dense = report_time("dense", timeit.repeat(lambda: run(dense_block), repeat=args.repeats, number=1), args.n, args.m, args.v)
    timeit.repeat(lambda: run(sparse_block), repeat=5, number=1)
    t_sparse = report_time("n:m", timeit.repeat(lambda: run(sparse_block), repeat=args.repeats, number=1), args.n, args.m, args.v)
    how = (" (fused feed-forward%s)" % (", activation in the kernel" if args.kernel_gelu else "")) if args.fuse_ffn else ""
    print("# dense %.2f ms, %d:%d:%d%s %.2f ms, speed-up %.2fx" % (t_dense, args.v, args.n, args.m, how, t_sparse, t_dense / t_sparse))


if __name__ == "__main__":
    main()
