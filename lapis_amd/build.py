"""Builds the gfx950 kernel library and the generated-module shim with hipcc.

Outputs (in-tree, next to this package, so that they travel with a source snapshot):
    lapis_amd/lib/liblapis_hip.so             the C-ABI kernel library (include/lapis_hip.h)
    lapis_amd/lib/liblapis_package_module.so  lapis_initialize / lapis_finalize / py_<func>
                                              (include/lapis_module.h), linked against the former
    lapis_amd/bin/lapis_spmv_bench            MatrixMarket SpMV benchmark driver (csrc/spmv_bench_main.cpp)

hipcc cross-compiles without a GPU.  Run ``python -m lapis_amd.build``.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(CSRC, "build")
INCLUDE = os.path.join(ROOT, "include")

KERNEL_SOURCES = ["runtime.hip", "spmv.hip", "colblock.hip", "colgroup.hip", "spmm.hip", "blas1.hip", "cg.hip",
                  "calibrate.hip"]
SHIM_SOURCES = ["module_shim.hip"]

KERNEL_LIB = os.path.join(LIBDIR, "liblapis_hip.so")
MODULE_LIB = os.path.join(LIBDIR, "liblapis_package_module.so")
BINDIR = os.path.join(HERE, "bin")
BENCH_BIN = os.path.join(BINDIR, "lapis_spmv_bench")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # separate multiply and add, as the reference's emitted C++ evaluates them
    "-ffp-contract=off",
    # no packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
    "-I", INCLUDE,
    "-I", CSRC,
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the kernel library cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + proc.stderr)
        raise RuntimeError("build step failed: " + os.path.basename(cmd[-1]))
    return proc.stdout + proc.stderr


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    _run([_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
    return obj


def build(verbose=False, jobs=8):
    """Compile every HIP source for gfx950 and link both shared libraries."""
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, KERNEL_SOURCES + SHIM_SOURCES))
    kobjs, sobjs = objs[: len(KERNEL_SOURCES)], objs[len(KERNEL_SOURCES):]
    _run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *kobjs, "-o", KERNEL_LIB])
    _run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *sobjs, "-L", LIBDIR, "-llapis_hip",
          "-Wl,-rpath,$ORIGIN", "-o", MODULE_LIB])
    os.makedirs(BINDIR, exist_ok=True)
    _run([_hipcc(), "--offload-arch=gfx950", "-O2", "-std=c++17", "-I", INCLUDE,
          os.path.join(CSRC, "spmv_bench_main.cpp"), "-L", LIBDIR, "-llapis_hip", "-Wl,-rpath,$ORIGIN/../lib", "-o",
          BENCH_BIN])
    if verbose:
        print("built", KERNEL_LIB)
        print("built", MODULE_LIB)
        print("built", BENCH_BIN)
    return KERNEL_LIB, MODULE_LIB


if __name__ == "__main__":
    build(verbose=True)
