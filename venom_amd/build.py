"""Build recipe of the native library (venom_amd/lib/libspatha.so) and of the
benchmark_spmm driver.

    python -m venom_amd.build          # compile everything for gfx950
    python -m venom_amd.build --ablation   # ... and the OUT_32B ablation variant of the library

Host-only sources go through g++ (OpenMP via libgomp), HIP sources through
hipcc --offload-arch=gfx950; hipcc links.  Everything is built in-tree.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
LIB = os.path.join(LIBDIR, "libspatha.so")
BENCH = os.path.join(LIBDIR, "benchmark_spmm")
TORCH_EXT = os.path.join(HERE, "_spatha_torch.so")       # the PyTorch C++ extension (operator `spmm`), importable in place

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed fp32 VALU ops are kept off for every device compile
HIP_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
CXX_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-fopenmp", "-Wall"]

# the SpMM kernels, one source per family (spmm_device.h holds what they share)
KERNEL_SOURCES = ["spmm_gathered.hip", "spmm_warpspec.hip", "spmm_densestage.hip", "spmm_unified.hip", "spmm_pingpong.hip",
                  "spmm_skinny.hip", "spmm_onehalf.hip"]
HIP_SOURCES = KERNEL_SOURCES + ["spmm_pack.hip", "spmm_dispatch.hip", "dense_gemm.hip", "transpose.hip", "layernorm.hip",
                                "select_gpu.hip", "spmm_static.hip", "spatha_api.cpp"]
CXX_SOURCES = ["vnm_format.cpp"]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def _compile_all(jobs, verbose):
    """Runs the compile commands side by side (the kernel file takes a minute, the others seconds)."""
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        for f in [pool.submit(_run, cmd, verbose) for cmd in jobs]:
            f.result()


def _torch_ext_compile():
    """g++ command for the PyTorch extension's only source (csrc/spatha_torch.cpp): written against the ROCm build of
    PyTorch directly, so it goes through the host compiler as it is."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension
    incs = cpp_extension.include_paths() + [sysconfig.get_paths()["include"], "/opt/rocm/include"]
    return (["g++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
             "-DTORCH_EXTENSION_NAME=_spatha_torch", "-DTORCH_API_INCLUDE_EXTENSION_H",
             "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)] +
            ["-isystem" + i for i in incs] +
            ["-c", os.path.join(CSRC, "spatha_torch.cpp"), "-o", os.path.join(OBJDIR, "spatha_torch.cpp.o")])


def _torch_ext_link(verbose):
    from torch.utils import cpp_extension
    libdirs = cpp_extension.library_paths()
    _run(["g++", "-shared", "-fPIC", "-o", TORCH_EXT, os.path.join(OBJDIR, "spatha_torch.cpp.o"), "-L" + LIBDIR, "-lspatha",
          "-Wl,-rpath,$ORIGIN/lib"] + ["-L" + d for d in libdirs] + ["-Wl,-rpath," + d for d in libdirs] +
         ["-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python"], verbose)
    return TORCH_EXT


def build(verbose=False, with_driver=True, with_out_32b=False, with_torch_ext=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    objs, jobs = [], []
    if with_torch_ext:
        jobs.append(_torch_ext_compile())
    for src in CXX_SOURCES:
        obj = os.path.join(OBJDIR, src + ".o")
        jobs.append(["g++"] + CXX_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    for src in HIP_SOURCES:
        obj = os.path.join(OBJDIR, src + ".o")
        lang = ["-x", "hip"] if src.endswith(".hip") else []
        jobs.append([HIPCC] + HIP_FLAGS + lang + ["-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    if with_out_32b:
        jobs += _out_32b_compile()
    _compile_all(jobs, verbose)
    if with_out_32b:
        _out_32b_link(verbose)
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs + ["-lgomp"], verbose)
    if with_driver and os.path.exists(os.path.join(CSRC, "benchmark_spmm.cpp")):
        # the driver alone links the vendor GEMM (hipBLASLt), the baseline of its gemm_time / speedup columns
        _run([HIPCC] + HIP_FLAGS + [os.path.join(CSRC, "benchmark_spmm.cpp"), os.path.join(CSRC, "vendor_gemm.cpp"), "-o", BENCH,
                                    "-L" + LIBDIR, "-lspatha", "-Wl,-rpath,$ORIGIN", "-L/opt/rocm/lib", "-lhipblaslt", "-lgomp"],
             verbose)
    if with_torch_ext:
        _torch_ext_link(verbose)
    build_calibrate(verbose)
    return LIB


def build_calibrate(verbose=False):
    """The machine calibration kernels of `bench.py --calibrate` (csrc/calibrate.hip): a library of their own,
    venom_amd/lib/libspatha_calibrate.so, so that the SpMM library exports the SpMM interface only."""
    lib = os.path.join(LIBDIR, "libspatha_calibrate.so")
    _run([HIPCC] + HIP_FLAGS + ["-x", "hip", "-shared", os.path.join(CSRC, "calibrate.hip"), "-o", lib], verbose)
    return lib


def build_variant(tag, defines, verbose=False, only=None):
    """A development build of the library with extra -D switches on the kernel sources (e.g. the timing knobs of
    spmm_pingpong.hip, SPATHA_UP_KNOBS=<bits>) -> venom_amd/lib/libspatha_<tag>.so; `SPATHA_LIBRARY=<that file>` makes the
    Python binding and bench.py load it.  Needs the objects of a normal build.  Such builds compute wrong results on
    purpose (a knob removes part of the kernel's work) and are for timing and power measurements only.  `only` names the
    sources that see the switches (default: all kernel sources; spatha_api.cpp, which reads the environment knobs of
    -DSPATHA_DEV_PROFILE builds, has to be named)."""
    sources = [src for src in HIP_SOURCES if src in only] if only else list(KERNEL_SOURCES)
    jobs = [[HIPCC] + HIP_FLAGS + ["-D" + d for d in defines] +
            ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", os.path.join(OBJDIR, "%s.%s.o" % (src, tag))] for src in sources]
    _compile_all(jobs, verbose)
    lib = os.path.join(LIBDIR, "libspatha_%s.so" % tag)
    objs = [os.path.join(OBJDIR, s + (".%s.o" % tag if s in sources else ".o")) for s in CXX_SOURCES + HIP_SOURCES]
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", lib] + objs + ["-lgomp"], verbose)
    return lib


def build_out_32b(verbose=False):
    """The OUT_32B ablation build (the reference's compile-time switch of that name, CMakeLists.txt:25-33): the same
    library with every 16-byte row-major store of C issued as four 4-byte stores -> venom_amd/lib/libspatha_out32b.so.
    Needs the objects of a normal build; `SPATHA_LIBRARY=<that file>` makes the Python binding load it."""
    _compile_all(_out_32b_compile(), verbose)
    return _out_32b_link(verbose)


def _out_32b_compile():
    return [[HIPCC] + HIP_FLAGS + ["-DSPATHA_OUT_32B", "-x", "hip", "-c", os.path.join(CSRC, src), "-o",
                                   os.path.join(OBJDIR, src + ".out32b.o")] for src in KERNEL_SOURCES]


def _out_32b_link(verbose):
    lib = os.path.join(LIBDIR, "libspatha_out32b.so")
    objs = [os.path.join(OBJDIR, s + (".out32b.o" if s in KERNEL_SOURCES else ".o")) for s in CXX_SOURCES + HIP_SOURCES]
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", lib] + objs + ["-lgomp"], verbose)
    return lib


if __name__ == "__main__":
    # python -m venom_amd.build [--ablation]            the library, the driver, the PyTorch extension (+ the OUT_32B build)
    # python -m venom_amd.build --variant TAG [--only SRC.hip] -DX=1 ...  a development build libspatha_TAG.so (after a normal build)
    argv = sys.argv[1:]
    if "--variant" in argv:
        only = [argv[i + 1] for i, a in enumerate(argv) if a == "--only"]
        build_variant(argv[argv.index("--variant") + 1], [a[2:] for a in argv if a.startswith("-D")], verbose=True, only=only)
    else:
        build(verbose=True, with_out_32b="--ablation" in argv)
    sys.exit(0)
