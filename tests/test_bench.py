"""bench.py: its bookkeeping on the CPU, and one short run of the whole script on the GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_algorithmic_bytes_of_the_headline_workload():
    # values 4096*256*2 + metadata 2048*32*4 + column-loc 64*128*16 + B 1024*16384*2 + C 4096*16384*2
    assert bench.algorithmic_bytes(4096, 1024, 16384, 8, 64, 256) == 2097152 + 262144 + 131072 + 33554432 + 134217728 == 170262528


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 2 and "one GPU only" in r.stderr and r.stdout == ""


def test_power_tool_output_is_parsed():
    text = json.dumps({"gpu_data": [{"gpu": 0, "power": {"socket_power": {"value": 1320, "unit": "W"}, "gfx_voltage": "N/A"},
                                     "clock": {"gfx_0": {"clk": {"value": 2000, "unit": "MHz"}, "min_clk": {"value": 500, "unit": "MHz"}},
                                               "gfx_1": {"clk": {"value": 2100, "unit": "MHz"}, "min_clk": {"value": 500, "unit": "MHz"}},
                                               "mem_0": {"clk": {"value": 2000, "unit": "MHz"}}}}]}, indent=4)
    assert bench.parse_smi(text) == (1320, 2050.0)
    assert bench.parse_smi("") is None and bench.parse_smi('{"error": "no devices"}') is None
    got = bench.smi_sample()            # whatever this machine has: a reading or nothing, never an exception
    assert got is None or (isinstance(got[0], int) and got[1] > 0)


def test_no_power_sampling_under_a_profiler(monkeypatch):
    for k in [k for k in os.environ if k.startswith(("ROCPROF", "ROCP_"))]:
        monkeypatch.delenv(k)
    monkeypatch.setenv("LD_PRELOAD", "/somewhere/libother.so")
    assert not bench.under_profiler()
    monkeypatch.setenv("LD_PRELOAD", "/opt/rocm/lib/librocprofiler-sdk-tool.so")
    assert bench.under_profiler()
    monkeypatch.setenv("LD_PRELOAD", "")
    monkeypatch.setenv("ROCPROF_OUTPUT_PATH", "/tmp/x")
    assert bench.under_profiler()


@pytest.mark.gpu
def test_short_run_prints_one_line_with_roofline_power_and_calibration():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "5", "--warmup", "2", "--settle-ms", "0",
                        "--no-extra", "--no-e2e", "--no-cpu-baseline", "--power-seconds", "0.6", "--calibrate"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [x for x in r.stdout.splitlines() if x.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    assert out["n_gpus"] == 1 and out["steps"] == 5 and out["warmup"] == 2 and out["vs_baseline"] is None
    roof = out["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["algorithmic_bytes"] == 170262528
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and 0.05 < roof["frac"] < 1.0
    assert abs(roof["achieved"] - roof["algorithmic_bytes"] / roof["kernel_us"] * 1e-3) < 1.0
    assert "power" in out            # a dict where amd-smi answers, else null
    if out["power"] is not None:
        assert out["power"]["us_per_spmm_sustained"] > 0
    cal = out["calibration"]
    assert set(cal) == {"store_c_alone", "smfmac_alone_gaussian", "smfmac32x32x32_alone_gaussian", "smfmac_alone_integers",
                        "smfmac_alone_zeros"}
    assert 1.0 < cal["store_c_alone"]["tb_per_s"] < 20.0
    # zeros are the cheapest operands: never slower than Gaussian ones, and never above the nominal peak
    assert cal["smfmac_alone_gaussian"]["pct_smfmac_peak"] <= cal["smfmac_alone_zeros"]["pct_smfmac_peak"] * 1.05 <= 105.0
    if out["power"] is not None and out["power"]["socket_w"]:
        pf = out["power_floor"]             # matrix instructions + C alone at the power limit: a floor, so below the kernel's time
        assert 0.2 < pf["frac"] < 1.05 and pf["matrix_mj"] > 0 and pf["store_mj"] > 0 and pf["limit_w"] > pf["idle_w"]


@pytest.mark.gpu
def test_default_run_carries_every_baseline_workload():
    """What the driver runs: one line with the headline figure, the other BASELINE workloads under `extra` (config 1, the 2:4
    baseline, 18 sweep cells, the GPT-3 matrix at three token counts), the encoder under `e2e`, the CPU baseline."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "20", "--warmup", "5", "--power-seconds", "0.6"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [x for x in r.stdout.splitlines() if x.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    extra = out["extra"]
    assert [e["config"][0] for e in extra] == ["1", "2"] + ["3"] * 18 + ["4"] * 3
    for e in extra:
        assert e["us"] > 0 and 0.02 < e["hbm_frac"] < 1.0 and e["bound"] in ("hbm", "mfma") and 0.05 < e["frac_of_bound"] < 1.0
        assert e["kernel"].startswith("smfmac16x16x64_")
    assert extra[0]["shape"] == "1024x4096x4096 128:2:8" and extra[0]["traffic"] is not None
    assert {e["shape"].split(" ")[1] for e in extra[2:20]} == {"%d:2:%d" % (v, m) for v in (64, 128) for m in (8, 16, 32)}
    assert [e["shape"].split("x")[2].split(" ")[0] for e in extra[20:]] == ["16", "256", "2048"]
    e2e = out["e2e"]
    assert e2e["format"] == "64:2:8" and e2e["layers"] == 24 and e2e["tokens"] == 16384
    assert e2e["dense_ms"] > e2e["vnm_ms"] > 0 and e2e["with_fused_blocks"]["vnm_ms"] < e2e["vnm_ms"]
    cpu = out["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and "bit-identical" in cpu["sample"]
