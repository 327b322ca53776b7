"""The reference's SpMM sweep over the BERT-base / BERT-large layer shapes (benchmark/run_spmm_spatha.sh): every
weight shape of the two models x N in {2048, 4096, 8192} tokens x V in {64, 128} x 2:M for M in {4, 7, 8, 10, 20, 40,
100}, each run through the `benchmark_spmm` driver with `--check`.  The reference tries a list of tile tuples per
point and keeps the best; here the library chooses the kernel (`--all-variants` tries every kernel id that fits
instead).  Writes the driver's CSV rows (the reference's 24 columns, then microseconds, dense-equivalent TFLOPS,
% of the sparse matrix-core peak, algorithmic GB/s, kernel name, host conversion seconds, host threads) under the
reference's header.

    python -m venom_amd.run_spmm_spatha [--out spmm_bert_spatha.csv] [--tokens 4096,8192] [--v 64,128] [--all-variants]
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


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default="spmm_bert_spatha.csv")
    ap.add_argument("--tokens", default="2048,4096,8192")
    ap.add_argument("--v", default="64,128")
    ap.add_argument("--m", default=",".join(str(x) for x in M_VALUES))
    ap.add_argument("--all-variants", action="store_true")
    args = ap.parse_args(argv)
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
