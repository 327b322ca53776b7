#!/usr/bin/env python3
"""Headline benchmark: V:N:M SpMM at 64:2:8 on the BERT-large FFN-up shape.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one SpMM  C[4096 x 16384] = A_vnm[4096 x 1024] * B[1024 x 16384]  (fp16 operands,
fp32 accumulation, fp16 result) with every operand already resident in HBM.  Prints ONE JSON
line: dense-equivalent TFLOPS (2*M*K*N / t), microseconds per SpMM, the roofline of the SpMM
kernel (HBM bound for this shape) and the CPU baseline (the CPU oracle's SpMM on a bounded
sample of the same workload, timed on this host's cores) and, where `amd-smi` answers, the socket power and graphics clock
under a sustained run of the same launches (`power`): on MI355X this kernel runs at the socket's power limit, which is what
sets its clock."""
import argparse
import ctypes
import json
import os
import re
import subprocess
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
SMFMAC_PEAK_TFLOPS = 5033.0    # fp16 MFMA with 2:4 structured sparsity (dense fp16 peak 2516.6 x 2)


# HBM-side bytes per launch of the default workload's kernel.  NOT measured by this script: the figure comes from two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE), each scaled by what the same counter reads for a
# plain 256 MiB device copy (--copy-calibration); the summary that holds it is named beside it and printed as
# roofline.traffic_source.  Keyed by kernel name and shape; any other kernel or shape reports null.
MEASURED_TRAFFIC = {
    ("smfmac16x16x64_warpspec_densestage_tile256x128_3stage_8consumers", 4096, 1024, 16384, 8, 64):
        (194_615_000, "profiles/spmm_ds_kernel_tile256x128_ffn_up_64-2-8.md"),
    ("smfmac16x16x64_unified_pingpong_densestage_aregs_tile512x128_3stage", 4096, 1024, 16384, 8, 64):
        (199_214_000, "profiles/spmm_up_kernel_tile512x128_ffn_up_64-2-8.md"),
    ("smfmac16x16x64_unified_pingpong_densestage_aregs_tile512x128_3stage", 4096, 1024, 16384, 4, 128):
        (271_000_000, "profiles/spmm_up_kernel_tile512x128_ffn_up_2-4.md"),
    ("smfmac16x16x64_warpspec_storewaves_tile128x128_3stage", 4096, 1024, 16384, 32, 128):
        (172_585_000, "profiles/spmm_wsw_kernel_tile128x128_ffn_up_128-2-32.md"),
    ("smfmac16x16x64_warpspec_storewaves_tile128x128_3stage", 1024, 4096, 4096, 8, 128):
        (61_530_000, "profiles/spmm_wsw_kernel_tile128x128_config1_128-2-8.md"),
    ("smfmac16x16x64_skinny_tile64xN_splitk4", 49152, 12288, 16, 16, 128):
        (184_100_000, "profiles/spmm_skinny_kernel_gpt3_ffn_n16.md"),
    ("smfmac16x16x64_warpspec_tile_and_a_half_192x256_4slots", 49152, 12288, 256, 16, 128):
        (251_500_000, "profiles/spmm_oh_kernel_gpt3_ffn_n256_128-2-16.md"),
    ("smfmac16x16x64_warpspec_tall_tile128x256_3stage", 49152, 12288, 2048, 16, 128):
        (2_202_100_000, "profiles/spmm_wst_kernel_tile128x256_gpt3_ffn_n2048.md"),
}


def smi_sample():
    """(socket power in W, mean graphics clock over the XCDs in MHz) from `amd-smi metric --power --clock --json`, or None."""
    try:
        r = subprocess.run(["amd-smi", "metric", "--power", "--clock", "--json"], capture_output=True, text=True, timeout=10)
    except (OSError, subprocess.SubprocessError):
        return None
    return parse_smi(r.stdout) if r.returncode == 0 else None


def parse_smi(text):
    """The two figures out of the tool's JSON text (one "socket_power" value, one "clk" value per "gfx_<n>" entry), or None."""
    watts = re.search(r'"socket_power": \{\s*"value": (\d+)', text)
    clocks = re.findall(r'"gfx_\d+": \{\s*"clk": \{\s*"value": (\d+)', text)
    if not watts or not clocks:
        return None
    return int(watts.group(1)), sum(map(int, clocks)) / len(clocks)


def under_profiler():
    """A profiler's preloaded library would load into the sampling tool as well: no power sampling under one."""
    return "rocprof" in os.environ.get("LD_PRELOAD", "") or any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ)


def sustained(launch, sync, us_estimate, seconds):
    """Back-to-back launches for `seconds` (after a quarter of that to settle) with `amd-smi` sampled from a second thread;
    returns (microseconds per launch by wall clock, mean socket W, mean gfx MHz, samples used) - power and clock None if
    the tool does not answer."""
    chunk = max(1, int(20e3 / max(us_estimate, 1.0)))          # synchronize every ~20 ms of queued work
    t_end = time.perf_counter() + seconds / 4
    while time.perf_counter() < t_end:
        for _ in range(chunk):
            launch()
        sync()
    samples, stop = [], threading.Event()

    def sampler():
        while not stop.is_set():
            got = smi_sample()
            if got is None:
                return
            samples.append((time.perf_counter(),) + got)
            stop.wait(0.15)

    th = threading.Thread(target=sampler)
    th.start()
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(chunk):
            launch()
        sync()
        n += chunk
    t1 = time.perf_counter()
    stop.set()
    th.join()
    used = [x for x in samples if t0 + min(0.8, seconds / 3) < x[0] < t1]      # the tool's reading lags by a few 100 ms
    if not used:
        return (t1 - t0) * 1e6 / n, None, None, 0
    return (t1 - t0) * 1e6 / n, sum(x[1] for x in used) / len(used), sum(x[2] for x in used) / len(used), len(used)


def algorithmic_bytes(rows, cols, N, m, v, ksp):
    """values + metadata + column-loc (as stored) + B read once + C written once."""
    return 2 * rows * ksp + 4 * (rows // 2) * (ksp // 8) + 16 * (rows // v) * (ksp // 2) + 2 * cols * N + 2 * rows * N


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20, help="untimed launches right before the timed ones")
    ap.add_argument("--settle-ms", type=float, default=200.0,
                    help="before the warm-up launches, keep launching the kernel for this many milliseconds: the GPU's clock "
                         "needs ~50-100 ms of work to settle, whatever --warmup says (reported as settle_ms, separate from warmup)")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the other BASELINE workloads that the default run reports under 'extra' (config 1, the 2:4 "
                         "baseline, the 18 cells of the sparsity sweep, the GPT-3 FFN matrix at 16 / 256 / 2048 tokens)")
    ap.add_argument("--rows", type=int, default=4096)
    ap.add_argument("--cols", type=int, default=1024)
    ap.add_argument("--n", type=int, default=16384, help="columns of B (tokens)")
    ap.add_argument("--m", type=int, default=8)
    ap.add_argument("--v", type=int, default=64)
    ap.add_argument("--variant", type=int, default=0)
    ap.add_argument("--value-std", type=float, default=0.02, help="standard deviation of A's non-zeros (BASELINE config 1: 1.0)")
    ap.add_argument("--b-uniform", action="store_true", help="B ~ U(-1, 1) instead of N(0, 1) (BASELINE config 1)")
    ap.add_argument("--split", action="store_true",
                    help="time the measured workload through spatha_spmm_run_ws (with a workspace: the library may split k-loops "
                         "over workgroups) instead of spatha_spmm_run")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--extra", action="store_true", help="also time three shapes outside BASELINE.json (appended to 'extra')")
    ap.add_argument("--ablation", action="store_true",
                    help="also time the same matrix with identity column-loc (the reference's IDEAL_KERNEL ablation) and, "
                         "if `python -m venom_amd.build --ablation` has been run, the OUT_32B build (4-byte stores of C)")
    ap.add_argument("--no-e2e", action="store_true",
                    help="skip the BERT-large encoder (BASELINE config 5: dense against 64:2:8 drop-in layers, under 'e2e'; "
                         "about a minute, most of it building and converting the model on the host)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="before the benchmark, run 5 plain device copies of 256 MiB (a kernel of known HBM traffic, "
                         "for scaling the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    ap.add_argument("--no-power", action="store_true",
                    help="skip the sustained run with `amd-smi` power / clock sampling that follows the timed region ('power')")
    ap.add_argument("--power-seconds", type=float, default=2.0, help="length of that sustained run")
    ap.add_argument("--no-calibrate", action="store_true",
                    help="skip the machine calibration kernels and the power floor derived from them ('calibration', 'power_floor'); "
                         "they run by default wherever power sampling works")
    ap.add_argument("--calibrate", action="store_true",
                    help="run the machine calibration kernels (venom_amd/csrc/calibrate.hip: a write of C alone, and sparse matrix "
                         "instructions alone on Gaussian / small-integer / zero operands; 'calibration') even where power sampling "
                         "does not work")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the SpMM path has no multi-GPU part); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    out32 = None
    if args.ablation and not os.environ.get("SPATHA_LIBRARY"):
        # the OUT_32B build of the library (python -m venom_amd.build --ablation), timed in a child process of its own
        # BEFORE this process touches the GPU
        alt = os.path.join(ROOT, "venom_amd", "lib", "libspatha_out32b.so")
        if os.path.exists(alt):
            import subprocess
            r = subprocess.run([sys.executable, os.path.abspath(__file__), "--no-cpu-baseline", "--no-extra", "--no-e2e", "--no-calibrate", "--steps", str(args.steps),
                                "--warmup", str(args.warmup), "--variant", str(args.variant)],
                               env=dict(os.environ, SPATHA_LIBRARY=alt), stdout=subprocess.PIPE, text=True)
            if r.returncode == 0 and r.stdout.strip():
                out32 = json.loads(r.stdout.strip().splitlines()[-1])["roofline"]["kernel_us"]

    idle = None if args.no_power or under_profiler() else smi_sample()

    import numpy as np
    import torch

    from venom_amd import _lib
    from venom_amd import format as F
    from venom_amd import spatha

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    L = _lib.lib()

    def prepare(rows, cols, N, m, v, seed=0, value_std=0.02, b_uniform=False):
        """Seeded synthetic operands: A's non-zeros ~ N(0, value_std); B ~ N(0, 1), or U(-1, 1) with b_uniform."""
        vals, meta, columns = F.synthetic_vnm(rows, cols, 2, m, v, seed=seed, value_std=value_std)
        g = F.geometry(rows, cols, 2, m, v)
        plan = spatha.SpmmPlan(torch.from_numpy(vals).to(dev), torch.from_numpy(meta.view(np.int32)).to(dev),
                               torch.from_numpy(columns.view(np.int32)).to(dev), rows, cols, 2, m, v)
        gen = torch.Generator(device=dev)
        gen.manual_seed(seed)
        if b_uniform:
            B = (torch.rand((cols, N), generator=gen, device=dev, dtype=torch.float32) * 2 - 1).to(torch.float16)
        else:
            B = torch.randn((cols, N), generator=gen, device=dev, dtype=torch.float32).to(torch.float16)
        C = torch.empty((rows, N), dtype=torch.float16, device=dev)
        return dict(vals=vals, meta=meta, columns=columns, geo=g, plan=plan, B=B, C=C)

    def timed(w, steps, warmup, variant=0, settle_ms=None):
        """Wall clock around `steps` launches bracketed by synchronize, plus HIP events on the
        launch stream over the same region (average kernel duration)."""
        plan, B, C = w["plan"], w["B"], w["C"]
        stream = torch.cuda.current_stream(dev)
        sp = ctypes.c_void_p(stream.cuda_stream)
        settle_ms = args.settle_ms if settle_ms is None else settle_ms
        if w.get("workspace") is not None:
            ws = w["workspace"]

            def launch():
                _lib.check(L.spatha_spmm_run_ws(plan._handle, B.data_ptr(), B.shape[1], None, C.data_ptr(), 0, 0, ws.data_ptr(),
                                                ws.numel(), sp), "run_ws")
        else:
            def launch():
                _lib.check(L.spatha_spmm_run(plan._handle, B.data_ptr(), B.shape[1], None, C.data_ptr(), 0, variant, sp), "run")
        t_settle = time.perf_counter()
        while (time.perf_counter() - t_settle) * 1e3 < settle_ms:       # time based: the clock settles on work done, not on a count
            for _ in range(20):
                launch()
            torch.cuda.synchronize()
        for _ in range(warmup):
            launch()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(steps):
            launch()
        e1.record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps

    if args.copy_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    rows, cols, N, m, v = args.rows, args.cols, args.n, args.m, args.v
    w = prepare(rows, cols, N, m, v, value_std=args.value_std, b_uniform=args.b_uniform)
    split_bytes = w["plan"].workspace_bytes(N) if args.split else 0
    if split_bytes:
        w["workspace"] = torch.zeros(split_bytes, dtype=torch.uint8, device=dev)
    ms_wall, ms_kernel = timed(w, args.steps, args.warmup, args.variant)
    ksp = w["geo"].ksp
    flops_dense = 2.0 * rows * cols * N
    flops_smfmac = 2.0 * rows * N * (2 * ksp)
    nbytes = algorithmic_bytes(rows, cols, N, m, v, ksp)
    tflops = flops_dense / (ms_wall * 1e-3) / 1e12
    achieved_gbs = nbytes / (ms_kernel * 1e-3) / 1e9

    traffic, traffic_source = MEASURED_TRAFFIC.get((w["plan"].kernel_name(N, 0, args.variant), rows, cols, N, m, v), (None, None))
    out = {
        "metric": "dense-equiv TFLOPS of the V:N:M SpMM at 64:2:8, BERT-large FFN",
        "value": round(tflops, 2),
        "unit": "TFLOPS (dense-equivalent, 2*M*K*N/t)",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": args.settle_ms,
        "ms_per_step": round(ms_wall, 6),
        "us_per_spmm": round(ms_wall * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 (fp32 accumulate)",
        "data": "synthetic (seed 0: A %d:2:%d random pattern, values ~N(0,%g); B ~%s)" % (v, m, args.value_std,
                                                                                            "U(-1,1)" if args.b_uniform else "N(0,1)"),
        "config": {"workload": "spmm A %dx%d %d:2:%d (Ksp %d) x B %dx%d, row-major C" % (rows, cols, v, m, ksp, cols, N),
                   "kernel": w["plan"].kernel_name(N, 0, args.variant),
                   "k_split_workspace_bytes": split_bytes},
        "pct_smfmac_peak": round(100.0 * flops_smfmac / (ms_kernel * 1e-3) / 1e12 / SMFMAC_PEAK_TFLOPS, 2),
        "roofline": {"bound": "hbm", "achieved": round(achieved_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved_gbs / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "algorithmic_bytes": nbytes, "kernel_us": round(ms_kernel * 1e3, 3)},
    }

    if idle is not None:
        # Sustained run of the same launches with the socket power and graphics clock sampled beside it.
        # (socket_w_at_start: the reading before this process touched the GPU - idle power, unless another run ended
        # within the last second or two.)
        stream = torch.cuda.current_stream(dev)
        sp = ctypes.c_void_p(stream.cuda_stream)
        plan, B, C = w["plan"], w["B"], w["C"]
        us_s, watts, mhz, n_s = sustained(
            lambda: _lib.check(L.spatha_spmm_run(plan._handle, B.data_ptr(), N, None, C.data_ptr(), 0, args.variant, sp), "run"),
            torch.cuda.synchronize, ms_kernel * 1e3, args.power_seconds)
        out["power"] = {"socket_w": None if watts is None else round(watts, 1), "gfx_mhz": None if mhz is None else round(mhz, 1),
                        "socket_w_at_start": idle[0], "us_per_spmm_sustained": round(us_s, 3),
                        "mj_per_spmm": None if watts is None else round(watts * us_s * 1e-3, 2), "samples": n_s,
                        "source": "amd-smi metric --power --clock, sampled over %.1f s of back-to-back launches after the timed "
                                  "region" % args.power_seconds}
    else:
        out["power"] = None

    if args.calibrate or (idle is not None and not args.no_calibrate):
        cal = ctypes.CDLL(os.path.join(ROOT, "venom_amd", "lib", "libspatha_calibrate.so"))
        cal.spatha_calibrate_store.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        cal.spatha_calibrate_smfmac.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                                ctypes.c_int, ctypes.c_void_p]
        stream = torch.cuda.current_stream(dev)
        sp = ctypes.c_void_p(stream.cuda_stream)
        wgs = torch.cuda.get_device_properties(dev).multi_processor_count
        calib = {}

        def run_cal(name, launch, us_guess, describe):
            us_c, watts, mhz, n_c = sustained(launch, torch.cuda.synchronize, us_guess, args.power_seconds)
            calib[name] = dict(describe(us_c), us=round(us_c, 2), socket_w=None if watts is None else round(watts, 1),
                               gfx_mhz=None if mhz is None else round(mhz, 1), samples=n_c)

        def check_hip(rc):
            if rc != 0:
                raise RuntimeError("calibration kernel: HIP error %d" % rc)

        c_rows, c_n = (rows // 512) * 512, (N // 128) * 128
        if c_rows and c_n:
            Cc = torch.empty((c_rows, c_n), dtype=torch.float16, device=dev)
            seed = [0]

            def launch_store():
                seed[0] += 1
                check_hip(cal.spatha_calibrate_store(Cc.data_ptr(), c_rows, c_n, wgs, seed[0], sp))

            run_cal("store_c_alone", launch_store, 20.0,
                    lambda us_c: {"bytes": 2 * c_rows * c_n, "tb_per_s": round(2 * c_rows * c_n / us_c * 1e-6, 2)})
            del Cc
        threads, passes = wgs * 512, 100
        gen = torch.Generator(device=dev)
        gen.manual_seed(1)
        out_c = torch.empty(threads, dtype=torch.float32, device=dev)
        operand_sets = {
            "smfmac_alone_gaussian": (torch.randn(threads * 32, generator=gen, device=dev) * 0.02,
                                      torch.randn(threads * 128, generator=gen, device=dev)),
            "smfmac_alone_integers": (torch.randint(-4, 5, (threads * 32,), generator=gen, device=dev).float(),
                                      torch.randint(-4, 5, (threads * 128,), generator=gen, device=dev).float()),
            "smfmac_alone_zeros": (torch.zeros(threads * 32, device=dev), torch.zeros(threads * 128, device=dev)),
        }
        for name, (a32, b32) in operand_sets.items():
            a16, b16 = a32.to(torch.float16), b32.to(torch.float16)
            # the 16 x 16 x 64 instruction the kernels use; for Gaussian operands also 32 x 32 x 32 (half as many instructions)
            for shape in ((16, 32) if name.endswith("gaussian") else (16,)):
                n_inst = wgs * 8 * passes * (32 if shape == 16 else 16)
                flops = wgs * 8 * passes * 32 * 16 * 16 * 64 * 2
                run_cal(name if shape == 16 else name.replace("smfmac_", "smfmac32x32x32_"),
                        lambda: check_hip(cal.spatha_calibrate_smfmac(a16.data_ptr(), b16.data_ptr(), out_c.data_ptr(), wgs, passes, shape, sp)),
                        60.0, lambda us_c: {"wave_instructions": n_inst, "dense_equiv_tflops": round(flops / us_c * 1e-6, 1),
                                            "pct_smfmac_peak": round(100 * flops / us_c * 1e-6 / SMFMAC_PEAK_TFLOPS, 1)})
        out["calibration"] = calib
        # The floor the socket's power limit puts under this workload, from the parts measured alone just now: the energy above
        # idle of its matrix instructions (on Gaussian operands) and of writing C once, spent at (limit - idle) watts, the limit
        # being the highest sustained socket power seen in this run.  Operand movement (L2 -> CU, LDS) is NOT in it.
        g, st = calib.get("smfmac_alone_gaussian"), calib.get("store_c_alone")
        if g and st and g["socket_w"] and st["socket_w"] and out.get("power") and out["power"]["socket_w"]:
            idle_w = float(idle[0])
            limit_w = max([out["power"]["socket_w"]] + [c["socket_w"] for c in calib.values() if c["socket_w"]])
            n_inst = (rows // 16) * (N // 16) * (ksp // 32)
            e_mfma = (g["socket_w"] - idle_w) * g["us"] * n_inst / g["wave_instructions"]          # microjoules
            e_store = (st["socket_w"] - idle_w) * st["us"] * (2.0 * rows * N) / st["bytes"]
            floor_us = (e_mfma + e_store) / (limit_w - idle_w)
            out["power_floor"] = {"us": round(floor_us, 2), "frac": round(floor_us / (ms_kernel * 1e3), 3),
                                  "matrix_mj": round(e_mfma * 1e-3, 2), "store_mj": round(e_store * 1e-3, 2),
                                  "idle_w": idle_w, "limit_w": round(limit_w, 1),
                                  "what": "(energy above idle of this workload's sparse matrix instructions on Gaussian operands + of "
                                          "writing C once, each measured alone) / (highest sustained socket power of this run - idle); "
                                          "operand movement not included; frac = that floor / the kernel's time"}

    def side_figures(r2, c2, n2, m2, v2, w2, k2, config):
        by = algorithmic_bytes(r2, c2, n2, m2, v2, w2["geo"].ksp)
        fl = 2.0 * r2 * n2 * 2 * w2["geo"].ksp
        t_hbm, t_mma = by / (HBM_PEAK_GBS * 1e9), fl / (SMFMAC_PEAK_TFLOPS * 1e12)
        tr, src = MEASURED_TRAFFIC.get((w2["plan"].kernel_name(n2, 0, 0), r2, c2, n2, m2, v2), (None, None))
        return {"config": config, "shape": "%dx%dx%d %d:2:%d" % (r2, c2, n2, v2, m2), "kernel": w2["plan"].kernel_name(n2, 0, 0),
                "algorithmic_bytes": by, "traffic": tr, "traffic_source": src,
                "us": round(k2 * 1e3, 2), "dense_equiv_tflops": round(2.0 * r2 * c2 * n2 / (k2 * 1e-3) / 1e12, 1),
                "hbm_gbs": round(by / (k2 * 1e-3) / 1e9, 1), "hbm_frac": round(by / (k2 * 1e-3) / 1e9 / HBM_PEAK_GBS, 3),
                "pct_smfmac_peak": round(100 * fl / (k2 * 1e-3) / 1e12 / SMFMAC_PEAK_TFLOPS, 2),
                "bound": "mfma" if t_mma > t_hbm else "hbm",
                "frac_of_bound": round(max(t_hbm, t_mma) / (k2 * 1e-3), 3)}

    def power_of(w2, n2, us_guess, seconds=1.5):
        """Socket power and clock under a sustained run of this workload (the compute-bound ones sit at the power limit)."""
        if idle is None:
            return None
        sp2 = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        plan2, B2, C2 = w2["plan"], w2["B"], w2["C"]
        us_s, watts, mhz, n_s = sustained(
            lambda: _lib.check(L.spatha_spmm_run(plan2._handle, B2.data_ptr(), n2, None, C2.data_ptr(), 0, 0, sp2), "run"),
            torch.cuda.synchronize, us_guess, seconds)
        return {"socket_w": None if watts is None else round(watts, 1), "gfx_mhz": None if mhz is None else round(mhz, 1),
                "us_sustained": round(us_s, 2), "samples": n_s}

    if not args.no_extra:
        # Every other workload BASELINE.json names, so that one default run carries them all (each: 100 ms settle, 10 warm-up,
        # 30 timed launches, HIP events): config 1 (the reference README's --check case with its own data), config 2 (2:4 on
        # the FFN-up shape), the 18 cells of config 3's sweep, config 4's three token counts.
        extra = []
        w2 = prepare(1024, 4096, 4096, 8, 128, value_std=1.0, b_uniform=True)
        _, k2 = timed(w2, 100, 20, settle_ms=100.0)
        e = side_figures(1024, 4096, 4096, 8, 128, w2, k2, "1: reference README case, A ~N(0,1), B ~U(-1,1)")
        e["vs_published_rtx3090_209.9us"] = round(209.9 / (k2 * 1e3), 2)
        extra.append(e)
        del w2
        w2 = prepare(4096, 1024, 16384, 4, 128)
        _, k2 = timed(w2, 30, 10, settle_ms=100.0)
        e = side_figures(4096, 1024, 16384, 4, 128, w2, k2, "2: plain 2:4 on the FFN-up shape")
        e["power"] = power_of(w2, 16384, k2 * 1e3)
        extra.append(e)
        del w2
        for (r2, c2) in ((1024, 1024), (4096, 1024), (1024, 4096)):
            for v2 in (64, 128):
                for m2 in (8, 16, 32):
                    if (r2, c2, m2, v2) == (rows, cols, m, v) and N == 16384 and args.variant == 0 and args.value_std == 0.02 \
                            and not args.b_uniform:
                        w2, k2 = w, ms_kernel               # the headline cell: measured above
                    else:
                        w2 = prepare(r2, c2, 16384, m2, v2)
                        _, k2 = timed(w2, 30, 10, settle_ms=100.0)
                    extra.append(side_figures(r2, c2, 16384, m2, v2, w2, k2, "3: sparsity sweep"))
                    w2 = None
        r2, c2, m2, v2 = 49152, 12288, 16, 128
        w2 = prepare(r2, c2, 16, m2, v2)
        for n2 in (16, 256, 2048):
            gen = torch.Generator(device=dev)
            gen.manual_seed(0)
            w2["B"] = torch.randn((c2, n2), generator=gen, device=dev, dtype=torch.float32).to(torch.float16)
            w2["C"] = torch.empty((r2, n2), dtype=torch.float16, device=dev)
            _, k2 = timed(w2, 30, 10, settle_ms=100.0)
            e = side_figures(r2, c2, n2, m2, v2, w2, k2, "4: GPT-3 FFN matrix, %d tokens" % n2)
            if n2 == 2048:
                e["power"] = power_of(w2, n2, k2 * 1e3)
            extra.append(e)
        del w2
        out["extra"] = extra

    if args.extra:
        extra = out.get("extra", [])
        for (r2, c2, n2, m2, v2) in [(1024, 4096, 4096, 8, 64), (4096, 1024, 16384, 4, 64), (1024, 4096, 4096, 8, 32)]:
            w2 = prepare(r2, c2, n2, m2, v2)
            _, k2 = timed(w2, 100, 20, settle_ms=100.0)
            extra.append(side_figures(r2, c2, n2, m2, v2, w2, k2, "other"))
            del w2
        out["extra"] = extra

    if not args.no_extra:
        # the k-split (spatha_spmm_run_ws): few tiles with long k-loops, here 128 tiles of 128 k-steps on the chip's CUs
        r2, c2, n2, m2, v2 = 1024, 16384, 1024, 8, 128
        w2 = prepare(r2, c2, n2, m2, v2)
        _, k_plain = timed(w2, 50, 10, settle_ms=50.0)
        need = w2["plan"].workspace_bytes(n2)
        ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=dev)
        sp2 = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

        def run_split():
            _lib.check(L.spatha_spmm_run_ws(w2["plan"]._handle, w2["B"].data_ptr(), n2, None, w2["C"].data_ptr(), 0, 0, ws.data_ptr(),
                                            need, sp2), "run_ws")

        for _ in range(20):
            run_split()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(50):
            run_split()
        e1.record()
        torch.cuda.synchronize()
        out["ksplit"] = {"shape": "%dx%dx%d %d:2:%d" % (r2, c2, n2, v2, m2), "kernel": w2["plan"].kernel_name(n2, 0, 0),
                         "unsplit_us": round(k_plain * 1e3, 2), "split_us": round(e0.elapsed_time(e1) / 50 * 1e3, 2),
                         "workspace_bytes": need,
                         "what": "k-loops of the 128 tiles in parts over the CUs that tiles alone leave idle (spatha_spmm_run_ws)"}
        del w2, ws

    if not args.no_e2e:
        # config 5: the BERT-large encoder, batch 32 x 512 tokens, every encoder Linear in 64:2:8 through the operator
        # (drop-in layers), against the same model on dense fp16 weights (hipBLASLt through torch)
        from venom_amd import bert
        torch.cuda.empty_cache()
        t_e2e = time.perf_counter()
        out["e2e"] = dict(bert.measure(n=2, m=8, v=64, repeats=10, warmups=3),
                          config="5: BERT-large encoder, 24 layers, batch 32 x seq 512, random-init weights, 64:2:8 drop-in layers")
        # ... and with the library's own additions to that path: feed-forward blocks without the transposed copy of the
        # [tokens, 4*hidden] activation (bias + GELU in the SpMM's write-out), the three attention projections as one SpMM,
        # residual + LayerNorm as one kernel (that one in the DENSE model as well: it does not depend on the weight format)
        torch.cuda.empty_cache()
        out["e2e"]["with_fused_blocks"] = dict(
            bert.measure(n=2, m=8, v=64, repeats=10, warmups=3, fuse_ffn=True, merge=True, fuse_ln=True, kernel_gelu=True,
                         ln_feature_major=True),
            what="fused feed-forward (bias + GELU in the write-out), merged q/k/v projections, residual + LayerNorm kernel in both "
                 "models; in the V:N:M model that kernel also writes the feature-major copy the next projection reads")
        out["e2e"]["wall_s_incl_model_build"] = round(time.perf_counter() - t_e2e, 1)

    if args.ablation:
        # the reference's IDEAL_KERNEL switch (CMakeLists.txt:25-33, blockwise_kernel.h): column-loc ignored, i.e. the
        # four gathered rows of every group are its first four -> the cost of the indirection is the difference
        ident = np.tile(np.arange(4, dtype=np.uint32), w["columns"].size // 4)
        w_id = dict(w)
        w_id["plan"] = spatha.SpmmPlan(torch.from_numpy(w["vals"]).to(dev), torch.from_numpy(w["meta"].view(np.int32)).to(dev),
                                       torch.from_numpy(ident.view(np.int32)).to(dev), rows, cols, 2, m, v)
        _, k_id = timed(w_id, args.steps, args.warmup, args.variant)
        _, k_nm = timed(w, args.steps, args.warmup, args.variant)
        out["ablation"] = {"column_loc_us": round(k_nm * 1e3, 2), "ideal_identity_column_loc_us": round(k_id * 1e3, 2),
                           "out_32b_stores_us": out32}      # null: libspatha_out32b.so has not been built

    if not args.no_cpu_baseline:
        import oracle

        threads = min(oracle.num_threads(), os.cpu_count() or 1)
        # whole workload, all cores: the oracle's compressed-form SpMM (fp32 accumulate, fp16 out)
        Bh = w["B"].cpu().numpy()
        reps = 0
        t0 = time.perf_counter()
        while True:
            ref = oracle.spmm(w["vals"], w["meta"], w["columns"], rows, cols, 2, m, v, Bh, threads=threads)
            reps += 1
            if time.perf_counter() - t0 > 4.0 or reps >= 20:
                break
        t_spmm = (time.perf_counter() - t0) / reps
        # one thread on an eighth of the columns
        n1 = max(8, (N // 8) // 8 * 8)
        t0 = time.perf_counter()
        oracle.spmm(w["vals"], w["meta"], w["columns"], rows, cols, 2, m, v, np.ascontiguousarray(Bh[:, :n1]), threads=1)
        t_one = (time.perf_counter() - t0) * (N / n1)
        # host format conversion of the same matrix, the reference's single-threaded way: decode + encode
        t0 = time.perf_counter()
        dense = oracle.decode(w["vals"], w["meta"], w["columns"], rows, cols, 2, m, v)
        oracle.encode(dense, w["columns"], 2, m, v)
        t_fmt = time.perf_counter() - t0
        got = w["C"].cpu().numpy()
        # |got - ref| / max(|ref|, rms(ref) / 16): relative to the entry unless it is far below the result's typical size
        err, same = 0.0, 0
        floor = max(float(np.sqrt(np.mean(ref[:256].astype(np.float64) ** 2))) / 16.0, 2.0 ** -14)
        for r0 in range(0, rows, 512):
            g64, r64 = got[r0:r0 + 512].astype(np.float64), ref[r0:r0 + 512].astype(np.float64)
            err = max(err, float(np.max(np.abs(g64 - r64) / np.maximum(np.abs(r64), floor))))
            same += int(np.count_nonzero(got[r0:r0 + 512].view(np.uint16) == ref[r0:r0 + 512].view(np.uint16)))
        out["cpu_baseline"] = {
            "value": round(flops_dense / t_spmm / 1e12, 5),
            "unit": "TFLOPS (dense-equivalent)",
            "cores": threads,
            "kind": "port",
            "sample": "oracle SpMM (compressed form, fp32 accumulate, OpenMP, %d threads) on the whole workload, mean of %d runs: "
                      "%.3f s per SpMM; 1 thread (timed on %d of %d columns, scaled): %.2f s; host format decode+encode of A, "
                      "1 thread: %.3f s; GPU vs oracle over all of C: max rel err %.2e (|d| / max(|ref|, rms/16)), %.4f of the "
                      "entries bit-identical" % (threads, reps, t_spmm, n1, N, t_one, t_fmt, err, same / float(rows * N)),
        }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
