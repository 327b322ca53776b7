"""The reference's two ablation sweeps (benchmark/run_ablation1.sh, benchmark/run_ablation2.sh) on one GPU.

ablation 1: what the column-loc indirection costs.  A 1024 x K x 4096 for K = 768 .. 12288 in steps of 768, V = 128,
    2:M for M in {10, 20, 40, 100}: the library as it is (algo 2) against the same matrices with identity column-loc,
    i.e. every group keeps its first four columns (algo 7; the reference's compile-time IDEAL_KERNEL switch,
    CMakeLists.txt:25-33).
ablation 2: what 16-byte stores of C are worth.  A 1024 x 4096 x 4096, V in {32, 64, 128}, M in {7, 8, 10, 20, 40, 100}:
    the library as it is (algo 2) against the OUT_32B build (algo 4; `python -m venom_amd.build --ablation`), which
    issues every row-major store of C as four 4-byte stores.

Rows follow the reference's header (tile columns 0: the library chooses the kernel; gemm_time and speedup 0: no dense
run here) with microseconds and the kernel's name appended.  `error` is 0 when the OUT_32B result has the same bits
as the normal build's (a checksum over C; ablation 1 changes the matrix, so there is nothing to compare).  Each
library is loaded in a process of its own; this process never touches the GPU.

    python -m venom_amd.run_ablation [--which 1,2] [--out-dir .] [--limit N]
"""
import argparse
import json
import os
import subprocess
import sys

HEADER = ("algo,arch,m,k,n,meta_block_sz,block_sz,nn_row,mm_row,density,bm,bn,bk,wm,wn,wk,mm,mn,mk,nstage,"
          "spmm_time,gemm_time,speedup,error,spmm_us,kernel")
ABLATION1_K = [768 * i for i in range(1, 17)]             # run_ablation1.sh:12-28
ABLATION1_M = [10, 20, 40, 100]
ABLATION2_V = [32, 64, 128]
ABLATION2_M = [7, 8, 10, 20, 40, 100]


def points(which, limit=0):
    if which == 1:
        pts = [(1024, k, 4096, 128, m) for m in ABLATION1_M for k in ABLATION1_K]
    else:
        pts = [(1024, 4096, 4096, v, m) for m in ABLATION2_M for v in ABLATION2_V]
    return pts[:limit] if limit else pts


def worker(which, ideal, limit=0):
    """Times every point of one sweep with the library this process loads; one JSON line per point on stdout."""
    import numpy as np
    import torch
    from . import format as F, spatha
    dev = torch.device("cuda:0")
    for rows, cols, N, v, m in points(which, limit):
        vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=0, value_std=0.02)
        if ideal:
            columns = np.tile(np.arange(4, dtype=np.uint32), columns.size // 4)
        plan = spatha.SpmmPlan(torch.from_numpy(vals).to(dev), torch.from_numpy(meta.view(np.int32)).to(dev),
                               torch.from_numpy(columns.view(np.int32)).to(dev), rows, cols, 2, m, v)
        gen = torch.Generator(device=dev)
        gen.manual_seed(0)
        B = torch.randn((cols, N), generator=gen, device=dev, dtype=torch.float32).to(torch.float16)
        C = torch.empty((rows, N), dtype=torch.float16, device=dev)
        plan.time(B, C, warmup=100, iters=100)
        ms = min(plan.time(B, C, warmup=10, iters=100) for _ in range(3))        # 10 + 100 launches as in the reference
        checksum = int(C.view(torch.int16).to(torch.int64).sum().item())
        print(json.dumps({"rows": rows, "cols": cols, "N": N, "v": v, "m": m, "ms": ms, "checksum": checksum,
                          "kernel": plan.kernel_name(N)}), flush=True)


def spawn(which, ideal=False, library=None, limit=0):
    env = dict(os.environ)
    if library:
        env["SPATHA_LIBRARY"] = library
    cmd = [sys.executable, "-m", "venom_amd.run_ablation", "--worker", str(which)] + (["--ideal"] if ideal else []) + \
          ["--limit", str(limit)]
    r = subprocess.run(cmd, env=env, capture_output=True, text=True, timeout=1200,
                       cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    if r.returncode != 0:
        raise RuntimeError("worker failed (%d): %s" % (r.returncode, r.stderr.strip()[-500:]))
    return [json.loads(ln) for ln in r.stdout.splitlines() if ln.startswith("{")]


def csv_row(algo, p, error):
    return "%d,gfx950,%d,%d,%d,32,4,2,%d,0.5,%d,0,0,0,0,0,0,0,0,0,%g,0,0,%d,%.3f,%s" % (
        algo, p["rows"], p["cols"], p["N"], p["m"], p["v"], p["ms"], error, p["ms"] * 1e3, p["kernel"])


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--which", default="1,2")
    ap.add_argument("--out-dir", default=".")
    ap.add_argument("--limit", type=int, default=0, help="only the first LIMIT points of each sweep (0 = all)")
    ap.add_argument("--worker", type=int, default=0, help=argparse.SUPPRESS)
    ap.add_argument("--ideal", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args(argv)
    if args.worker:
        worker(args.worker, args.ideal, args.limit)
        return 0
    from . import _lib
    status = 0
    for which in [int(x) for x in args.which.split(",")]:
        base = spawn(which, limit=args.limit)
        if which == 1:
            other, algo = spawn(1, ideal=True, limit=args.limit), 7
        else:
            lib32 = os.path.join(os.path.dirname(_lib.LIB_PATH), "libspatha_out32b.so")
            if not os.path.exists(lib32):
                raise RuntimeError("libspatha_out32b.so is not built: run `python -m venom_amd.build --ablation`")
            other, algo = spawn(2, library=lib32, limit=args.limit), 4
        path = os.path.join(args.out_dir, "ablation%d.csv" % which)
        with open(path, "w") as f:
            f.write(HEADER + "\n")
            for p in base:
                f.write(csv_row(2, p, 0) + "\n")
            for p, q in zip(base, other):
                error = 0 if which == 1 or p["checksum"] == q["checksum"] else 1
                status |= error
                f.write(csv_row(algo, q, error) + "\n")
        for p, q in zip(base, other):
            print("%dx%dx%d %d:2:%d: %.1f us, %s %.1f us (%+.1f %%)" % (
                p["rows"], p["cols"], p["N"], p["v"], p["m"], p["ms"] * 1e3,
                "identity column-loc" if which == 1 else "4-byte stores", q["ms"] * 1e3, 100.0 * (q["ms"] / p["ms"] - 1)),
                flush=True)
    return status


if __name__ == "__main__":
    sys.exit(main())
