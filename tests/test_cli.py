"""The benchmark_spmm driver: flags, error behaviour and CSV row of the reference's driver
(src/benchmark_spmm.cpp:157-222, src/util/argparse.h:24-233).

Argument errors are raised before any device work, so those tests run without a GPU; the runs
themselves draw their inputs like the reference does (small integers from rand(): B, then the
pattern, then A's values) and are held to the reference's own acceptance rule through --check."""
import os
import subprocess

import numpy as np
import pytest

from venom_amd import format as F

BENCH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "venom_amd", "lib", "benchmark_spmm")

# README.md:174 of the reference (its worked example: 1024 x 4096 x 4096 at 128:2:8)
CONFIG1 = ("--sparsity-type n-to-m --spmm spatha --gemm cuBlas --precision half --meta-block-size 32 --block-size 4 "
           "--nn_row 2 --mm_row 8 --m 1024 --k 4096 --n 4096 --d 0.5 --bm 128 --bn 64 --bk 32 --wm 32 --wn 64 --wk 32 "
           "--mm 16 --mn 8 --mk 32 --nstage 2 --random --check").split()

REFERENCE_COLUMNS = ("algo,arch,m,k,n,meta_block_sz,block_sz,nn_row,mm_row,density,bm,bn,bk,wm,wn,wk,mm,mn,mk,nstage,"
                     "spmm_time,gemm_time,speedup,error").split(",")       # benchmark/run_ablation2.sh:12
APPENDED_COLUMNS = "spmm_us,dense_equiv_tflops,pct_smfmac_peak,hbm_gbs,kernel,cpu_encode_decode_s,cpu_threads,gemm_impl".split(",")


def _run(args, timeout=300):
    return subprocess.run([BENCH] + list(args), stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout)


def _replace(args, flag, value):
    out = list(args)
    out[out.index(flag) + 1] = str(value)
    return out


def _row(stdout):
    lines = [ln for ln in stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, stdout
    fields = lines[0].split(",")
    assert len(fields) == len(REFERENCE_COLUMNS) + len(APPENDED_COLUMNS)
    return dict(zip(REFERENCE_COLUMNS + APPENDED_COLUMNS, fields))


def test_driver_is_built():
    assert os.access(BENCH, os.X_OK)


@pytest.mark.parametrize("args,needle", [
    ([], "Forget to set m,n,k,density"),
    (["--m", "64"], "Forget to set m,n,k,density"),
    (CONFIG1 + ["--frobnicate"], "unknown or incomplete argument: --frobnicate"),
    (CONFIG1 + ["--m"], "unknown or incomplete argument: --m"),            # a value flag in last position
    (_replace(CONFIG1, "--d", 0), "Forget to set m,n,k,density"),         # --d must be non-zero, as in the reference
    (_replace(CONFIG1, "--sparsity-type", "csr"), "n-to-m"),
    (_replace(CONFIG1, "--spmm", "sputnik"), "spatha"),
    (_replace(CONFIG1, "--precision", "single"), "only precision:half is implemented"),
    (_replace(CONFIG1, "--precision", "int8"), "only precision:half is implemented"),
    (_replace(CONFIG1, "--nn_row", 1), "--nn_row must be 2"),
    (_replace(CONFIG1, "--mm_row", 3), "--mm_row >= 4"),
    (_replace(CONFIG1, "--m", 1000), "shape not representable"),          # rows % V
    (_replace(CONFIG1, "--bm", 48), "shape not representable"),           # V % 32
    (_replace(CONFIG1, "--n", 4100), "multiple of 8"),
    ([a for a in CONFIG1 if a not in ("--bm", "128")], "--bm (V) is required"),
])
def test_argument_errors_print_usage_and_exit_1(args, needle):
    r = _run(args, timeout=60)
    assert r.returncode == 1
    assert r.stdout == ""
    assert "Required cmdline args" in r.stderr and needle in r.stderr


@pytest.mark.gpu
def test_config1_invocation_passes_its_own_check(gpu):
    r = _run(CONFIG1)
    assert r.returncode == 0, r.stderr
    row = _row(r.stdout)
    assert row["algo"] == "2" and row["arch"] == "gfx950" and row["error"] == "0"
    assert [row[c] for c in ("m", "k", "n", "meta_block_sz", "block_sz", "nn_row", "mm_row", "density")] == \
        ["1024", "4096", "4096", "32", "4", "2", "8", "0.5"]
    # the NVIDIA tile flags are echoed, not interpreted
    assert [row[c] for c in ("bm", "bn", "bk", "wm", "wn", "wk", "mm", "mn", "mk", "nstage")] == \
        ["128", "64", "32", "32", "64", "32", "16", "8", "32", "2"]
    spmm_ms, gemm_ms, speedup = float(row["spmm_time"]), float(row["gemm_time"]), float(row["speedup"])
    assert 0 < spmm_ms < 1.0 and gemm_ms > 0 and abs(speedup - gemm_ms / spmm_ms) <= 1e-3 * speedup
    assert abs(float(row["spmm_us"]) - spmm_ms * 1e3) <= 0.01 * spmm_ms * 1e3 + 1e-3
    want_tflops = 2.0 * 1024 * 4096 * 4096 / (spmm_ms * 1e-3) / 1e12
    assert abs(float(row["dense_equiv_tflops"]) - want_tflops) <= 0.01 * want_tflops
    assert row["kernel"].startswith("smfmac16x16x64_")
    assert row["gemm_impl"] == "hipblaslt"            # the speed-up column is against the vendor library's dense GEMM


@pytest.mark.gpu
def test_tune_times_every_kernel_and_runs_the_fastest(gpu):
    """--tune: the times of the automatic choice and of every kernel id that takes the shape go to stderr, the fastest id
    runs the benchmark, and --check still holds."""
    r = _run(_replace(_replace(CONFIG1, "--n", 2048), "--m", 512) + ["--tune"])
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stderr.splitlines() if l.startswith("tune:")]
    assert len(lines) >= 3 and lines[0].startswith("tune: id  0 ")
    assert sum("<- fastest" in l for l in lines) == 1
    row = _row(r.stdout)
    assert row["error"] == "0"
    fastest = [l for l in lines if "<- fastest" in l][0]
    assert row["kernel"] in fastest


@pytest.mark.gpu
@pytest.mark.parametrize("m,k,n,mm_row,bm", [
    (256, 1000, 264, 10, 64),      # K % m == 0 but Ksp padded; ragged N
    (512, 330, 136, 7, 128),       # two-column tail group
    (128, 512, 72, 16, 32),        # V = 32
    (256, 256, 16, 4, 64),         # plain 2:4, few columns
    (192, 4096, 520, 32, 192),
])
def test_other_shapes_pass_the_check(gpu, m, k, n, mm_row, bm):
    args = CONFIG1
    for flag, value in (("--m", m), ("--k", k), ("--n", n), ("--mm_row", mm_row), ("--bm", bm)):
        args = _replace(args, flag, value)
    r = _run(args)
    assert r.returncode == 0, r.stderr
    row = _row(r.stdout)
    assert row["error"] == "0" and [row["m"], row["k"], row["n"], row["mm_row"], row["bm"]] == [str(x) for x in (m, k, n, mm_row, bm)]


@pytest.mark.gpu
def test_every_kernel_id_is_reachable_or_refused(gpu):
    """--variant picks the kernel; an id that does not fit the shape ends with a message, not a wrong result."""
    args = _replace(_replace(_replace(CONFIG1, "--m", 256), "--k", 512), "--n", 256)
    names = set()
    for variant in range(0, 40):
        r = _run(args + ["--variant", str(variant)])
        if r.returncode == 0:
            row = _row(r.stdout)
            assert row["error"] == "0"
            names.add(row["kernel"])
        else:
            assert r.returncode == 1 and r.stdout == "" and "does not support" in r.stderr
    assert len(names) >= 10


@pytest.mark.gpu
def test_path_to_dset_writes_then_reads_the_matrix(gpu, tmp_path):
    path = str(tmp_path / "a.vnm")
    args = _replace(_replace(_replace(CONFIG1, "--m", 256), "--k", 512), "--n", 128) + ["--path_to_dset", path]
    first = _run(args)
    assert first.returncode == 0, first.stderr
    vals, meta, cols, geo = F.load(path)
    assert (geo.rows, geo.cols, geo.n, geo.m, geo.v) == (256, 512, 2, 8, 128) and vals.dtype == np.float16
    # the stored matrix obeys the format: two kept values per group, values are the driver's small integers
    assert np.all(np.abs(vals.astype(np.float32)) <= 4) and np.all(vals.astype(np.float32) == np.round(vals.astype(np.float32)))
    # a second run reads it back (and still passes the check against the dense product of what it read)
    vals2 = (vals.astype(np.float32) * 0).astype(np.float16)
    vals2[::7] = np.float16(3.0)
    F.save(path, vals2, meta, cols, 256, 512, 2, 8, 128)
    second = _run(args)
    assert second.returncode == 0, second.stderr
    assert _row(second.stdout)["error"] == "0"
    # a container of another shape is refused
    third = _run(_replace(args, "--k", 1024))
    assert third.returncode == 1 and "--path_to_dset" in third.stderr


@pytest.mark.gpu
def test_out_32b_ablation_build_computes_the_same_numbers(gpu):
    """The OUT_32B build (4-byte stores of C) only changes how the result leaves the GPU."""
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    alt = os.path.join(root, "venom_amd", "lib", "libspatha_out32b.so")
    if not os.path.exists(alt):
        pytest.skip("libspatha_out32b.so has not been built (python -m venom_amd.build --ablation)")
    r = subprocess.run([sys.executable, "-c", "import __graft_entry__ as g; g.smoke()"], cwd=root,
                       env=dict(os.environ, SPATHA_LIBRARY=alt), stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                       timeout=300)
    assert r.returncode == 0 and "smoke ok" in r.stdout, r.stderr[-2000:]


def test_sweep_script_issues_the_reference_command_lines():
    """run_spmm_spatha builds, per point, the command line of benchmark/run_spmm_spatha.sh:135 (with --check)."""
    from venom_amd import run_spmm_spatha as sweep
    cmd = sweep.command(4096, 1024, 8192, 64, 7)
    assert cmd[0] == BENCH
    for flag, value in (("--sparsity-type", "n-to-m"), ("--spmm", "spatha"), ("--gemm", "cuBlas"), ("--precision", "half"),
                        ("--meta-block-size", "32"), ("--block-size", "4"), ("--nn_row", "2"), ("--mm_row", "7"),
                        ("--m", "4096"), ("--k", "1024"), ("--n", "8192"), ("--bm", "64")):
        assert cmd[cmd.index(flag) + 1] == value
    assert "--check" in cmd and "--variant" not in cmd
    assert sweep.command(64, 64, 64, 64, 4, variant=5)[-2:] == ["--variant", "5"]
    assert sweep.HEADER.split(",")[:24] == [c if c != "mm_row" else "mm_col" for c in REFERENCE_COLUMNS]   # run_spmm_spatha.sh:8
    assert len(sweep.HEADER.split(",")) == len(REFERENCE_COLUMNS) + len(APPENDED_COLUMNS)
    assert (768, 3072) in sweep.LAYERS and (4096, 1024) in sweep.LAYERS and sweep.M_VALUES == [4, 7, 8, 10, 20, 40, 100]


@pytest.mark.gpu
def test_sweep_script_runs_and_every_point_passes_the_check(gpu, tmp_path):
    from venom_amd import run_spmm_spatha as sweep
    out = str(tmp_path / "sweep.csv")
    assert sweep.main(["--out", out, "--tokens", "2048", "--v", "64,128", "--m", "7,20"]) == 0
    lines = open(out).read().splitlines()
    assert lines[0] == sweep.HEADER and len(lines) == 1 + 2 * 2 * len(sweep.LAYERS)
    for ln in lines[1:]:
        row = dict(zip(sweep.HEADER.split(","), ln.split(",")))
        assert row["error"] == "0" and row["arch"] == "gfx950" and float(row["spmm_time"]) > 0


def test_ablation_script_covers_the_reference_points():
    """run_ablation: the shapes of benchmark/run_ablation1.sh:12-28 (V = 128, M in 10, 20, 40, 100) and of
    run_ablation2.sh:8 (V in 32, 64, 128; M in 7 .. 100), rows under the reference's header."""
    from venom_amd import run_ablation as ab
    p1, p2 = ab.points(1), ab.points(2)
    assert len(p1) == 16 * 4 and {p[1] for p in p1} == {768 * i for i in range(1, 17)} and {p[3] for p in p1} == {128}
    assert len(p2) == 18 and {p[:3] for p in p2} == {(1024, 4096, 4096)} and {p[3] for p in p2} == {32, 64, 128}
    assert ab.points(2, limit=2) == p2[:2]
    assert ab.HEADER.split(",")[:24] == REFERENCE_COLUMNS
    row = ab.csv_row(4, {"rows": 1024, "cols": 4096, "N": 4096, "m": 8, "v": 64, "ms": 0.025, "kernel": "k"}, 0).split(",")
    assert len(row) == len(ab.HEADER.split(",")) and row[0] == "4" and row[8] == "8" and row[10] == "64" and row[23] == "0"


@pytest.mark.gpu
def test_ablation_script_runs_both_builds_and_they_agree(gpu, tmp_path):
    from venom_amd import run_ablation as ab
    assert ab.main(["--which", "2", "--limit", "3", "--out-dir", str(tmp_path)]) == 0
    lines = open(str(tmp_path / "ablation2.csv")).read().splitlines()
    assert lines[0] == ab.HEADER and len(lines) == 1 + 2 * 3
    assert [ln.split(",")[0] for ln in lines[1:]] == ["2"] * 3 + ["4"] * 3
    assert all(ln.split(",")[23] == "0" for ln in lines[1:])
