"""The host format builder under AddressSanitizer + UndefinedBehaviorSanitizer (CPU only): tests/sanitize_format_host.cpp
drives every entry point of venom_amd/csrc/vnm_format.cpp with exactly-sized buffers; a report from either sanitizer
aborts the run.  The sanitizer runtime is linked statically, so that it initialises first whatever the environment
preloads."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host compiler")
def test_format_builder_is_clean_under_asan_and_ubsan(tmp_path):
    exe = str(tmp_path / "sanitize_format_host")
    build = subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fopenmp", "-fsanitize=address,undefined",
                            "-fno-sanitize-recover=all", "-static-libasan",
                            os.path.join(HERE, "sanitize_format_host.cpp"),
                            os.path.join(ROOT, "venom_amd", "csrc", "vnm_format.cpp"), "-o", exe],
                           capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe, str(tmp_path)], capture_output=True, text=True, timeout=600, env=env)
    assert run.returncode == 0, (run.stdout[-1000:], run.stderr[-3000:])
    assert "sanitized host format builder: ok" in run.stdout
