"""The reference's SpMM sweep over the BERT-base / BERT-large layer shapes (benchmark/run_spmm_spatha.sh): every
weight shape of the two models x N in {2048, 4096, 8192} tokens x V in {64, 128} x 2:M for M in {4, 7, 8, 10, 20, 40,
100}, each run through the `benchmark_spmm` driver with `--check`.  The reference tries a list of tile tuples per
point and keeps the best; here the library chooses the kernel (`--all-variants` tries every kernel id that fits
instead).  Writes the driver's CSV rows (the reference's 24 columns, then microseconds, dense-equivalent TFLOPS,
% of the sparse matrix-core peak, algorithmic GB/s, kernel name, host conversion seconds, host threads) under the
reference's header.

    python -m venom_amd.run_spmm_spatha [--out spmm_bert_spatha.csv] [--tokens 4096,8192] [--v 64,128] [--all-variants]

`--compare-kernels` answers a different question on the same points, in this process and with Gaussian data: how far is
the library's automatic choice from the fastest kernel id that accepts the shape?  It times every id on every point
(HIP events, 2 x 40 launches each), writes one JSON line per point to --out and prints the points where the choice is
more than 5 % behind, then the geometric mean of automatic / best.
"""
import argparse
import os
import subprocess
import sys

from . import _lib

HEADER = ("algo,arch,m,k,n,meta_block_sz,block_sz,nn_row,mm_col,density,bm,bn,bk,wm,wn,wk,mm,mn,mk,nstage,"
          "spmm_time,gemm_time,speedup,error,spmm_us,tflops_dense_equiv,pct_sparse_peak,gbs,kernel,convert_s,threads,gemm_impl")
# (rows, cols) of the linear layers: BERT-base 768 / 3072, BERT-large 1024 / 4096 (run_spmm_spatha.sh:12-30)
LAYERS = [(768, 768), (3072, 768), (768, 3072), (1024, 1024), (4096, 1024), (1024, 4096)]
M_VALUES = [4, 7, 8, 10, 20, 40, 100]


def driver_path():
    path = os.path.join(os.path.dirname(_lib.LIB_PATH), "benchmark_spmm")
    if not os.path.exists(path):
        raise RuntimeError("benchmark_spmm is not built: run `python -m venom_amd.build`")
    return path


def command(rows, cols, tokens, v, m, variant=0):
    """The reference's command line for one point (tile arguments are accepted and ignored by this driver)."""
    cmd = [driver_path(), "--sparsity-type", "n-to-m", "--spmm", "spatha", "--gemm", "cuBlas", "--precision", "half",
           "--meta-block-size", "32", "--block-size", "4", "--nn_row", "2", "--mm_row", str(m), "--m", str(rows),
           "--k", str(cols), "--n", str(tokens), "--d", "0.5", "--bm", str(v), "--bn", "64", "--bk", "32",
           "--wm", "32", "--wn", "64", "--wk", "32", "--mm", "16", "--mn", "8", "--mk", "32", "--nstage", "2", "--check"]
    if variant:
        cmd += ["--variant", str(variant)]
    return cmd


def run_point(rows, cols, tokens, v, m, all_variants=False, num_variants=64):
    """Returns (csv_row or None, message).  With all_variants: the fastest row among the kernel ids that accept the shape."""
    best = None
    message = ""
    for variant in (range(1, num_variants) if all_variants else [0]):
        r = subprocess.run(command(rows, cols, tokens, v, m, variant), capture_output=True, text=True, timeout=300)
        if r.returncode == 1 and "does not support" in r.stderr:
            continue
        if r.returncode != 0 or not r.stdout.strip():
            message = "exit %d: %s" % (r.returncode, r.stderr.strip().splitlines()[-1] if r.stderr.strip() else "")
            if not all_variants:
                return None, message
            continue
        row = r.stdout.strip().splitlines()[-1]
        t = float(row.split(",")[20])
        if best is None or t < best[0]:
            best = (t, row)
    return (best[1], "") if best else (None, message or "no kernel accepted the shape")


def compare_kernels(out_path, tokens, vs, ms):
    """Automatic choice against the best kernel id, per point; returns the list of automatic / best ratios."""
    import json
    import math

    import numpy as np
    import torch

    from . import format as F
    from . import spatha

    ratios = []
    with open(out_path, "w") as f:
        for rows, cols in LAYERS:
            for v in vs:
                if rows % v:
                    continue
                for m in ms:
                    vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=0, value_std=0.02)
                    plan = spatha.SpmmPlan(torch.from_numpy(vals).cuda(), torch.from_numpy(meta.view(np.int32)).cuda(),
                                           torch.from_numpy(columns.view(np.int32)).cuda(), rows, cols, 2, m, v)
                    for N in tokens:
                        gen = torch.Generator(device="cuda")
                        gen.manual_seed(0)
                        B = torch.randn((cols, N), generator=gen, device="cuda").half()
                        out = torch.empty((rows, N), dtype=torch.float16, device="cuda")
                        auto = plan.kernel_name(N, 0, 0)
                        plan.time(B, out, warmup=30, iters=30)
                        times = {}
                        for variant in range(1, spatha.num_variants()):
                            name = plan.kernel_name(N, 0, variant)
                            if name is not None:
                                times[name] = min(plan.time(B, out, variant=variant, warmup=5, iters=40) for _ in range(2)) * 1e3
                        if auto not in times:       # not one kernel id: an uneven last round run as two launches
                            times[auto] = min(plan.time(B, out, variant=0, warmup=5, iters=40) for _ in range(2)) * 1e3
                        best = min(times, key=times.get)
                        ratio = times[auto] / times[best]
                        ratios.append(ratio)
                        f.write(json.dumps({"rows": rows, "cols": cols, "N": N, "v": v, "m": m, "auto": auto, "best": best,
                                            "ratio": round(ratio, 3), "us": {k: round(t, 2) for k, t in times.items()}}) + "\n")
                        f.flush()
                        if ratio > 1.05:
                            print("%dx%dx%d %d:2:%d: %s %.2f us, best %s %.2f us (%.3f)" %
                                  (rows, cols, N, v, m, auto, times[auto], best, times[best], ratio), flush=True)
    print("%d points: automatic / best, geometric mean %.4f; within 5 %%: %d, within 10 %%: %d, worst %.3f" %
          (len(ratios), math.exp(sum(math.log(r) for r in ratios) / len(ratios)), sum(r <= 1.05 for r in ratios),
           sum(r <= 1.10 for r in ratios), max(ratios)), flush=True)
    return ratios


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default="spmm_bert_spatha.csv")
    ap.add_argument("--tokens", default="2048,4096,8192")
    ap.add_argument("--v", default="64,128")
    ap.add_argument("--m", default=",".join(str(x) for x in M_VALUES))
    ap.add_argument("--all-variants", action="store_true")
    ap.add_argument("--compare-kernels", action="store_true",
                    help="time every kernel id on every point in this process (Gaussian data) and compare with the automatic choice")
    args = ap.parse_args(argv)
    if args.compare_kernels:
        compare_kernels(args.out if args.out != "spmm_bert_spatha.csv" else "spmm_bert_kernels.jsonl",
                        [int(x) for x in args.tokens.split(",")], [int(x) for x in args.v.split(",")],
                        [int(x) for x in args.m.split(",")])
        return 0
    failures = 0
    with open(args.out, "w") as f:
        f.write(HEADER + "\n")
        for m in [int(x) for x in args.m.split(",")]:
            for v in [int(x) for x in args.v.split(",")]:
                for tokens in [int(x) for x in args.tokens.split(",")]:
                    for rows, cols in LAYERS:
                        row, message = run_point(rows, cols, tokens, v, m, args.all_variants)
                        if row is None:
                            failures += 1
                            print("# %dx%dx%d %d:2:%d FAILED: %s" % (rows, cols, tokens, v, m, message), flush=True)
                            continue
                        f.write(row + "\n")
                        f.flush()
                        c = row.split(",")
                        print("%dx%dx%d %d:2:%d: %s us, %s TFLOPS dense-equivalent, error %s, %s" %
                              (rows, cols, tokens, v, m, c[24], c[25], c[23], c[28]), flush=True)
    return 1 if failures else 0


if __name__ == "__main__":
    sys.exit(main())
