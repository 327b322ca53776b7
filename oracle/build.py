"""Build recipe for the CPU oracle (test infrastructure only).

    python oracle/build.py

compiles oracle/vnm_oracle.cpp into oracle/libvnm_oracle.so with g++.  The
reference's own C++ host sources cannot be built in this image (they include
CUDA runtime headers that are absent, and writing stand-ins for them is not an
option), so there is no oracle/_ref build; the oracle is pinned by the golden
vectors under tests/golden and by the closed-form / brute-force checks in
tests/.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "vnm_oracle.cpp")
OUT = os.path.join(HERE, "libvnm_oracle.so")


def build(force=True, verbose=False):
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    cmd = ["g++", "-O3", "-std=c++17", "-fopenmp", "-fPIC", "-shared", "-o", OUT, SRC]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    build(force=True, verbose=True)
    sys.exit(0)
