"""Builds the HIP library (and, on request, the torch op registration layer)
in-tree.  Run as `python -m sonar_amd.build`."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libsonar_marlin.so")
OPS_PATH = os.path.join(LIB_DIR, "libsonar_marlin_torch.so")
BENCH_PATH = os.path.join(LIB_DIR, "libsonar_bench.so")   # bench.py's yardstick kernels, not part of the product
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

HIP_SOURCES = ["repack.hip", "gemm_stream.hip", "gemm_tile.hip", "gemm_moe.hip", "moe_aux.hip", "gemm_a8.hip", "quant_input.hip"]
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# The compiler the hand-scheduled kernels were checked with.  Their asm statements
# (loads whose results land many instructions later, tied to their use only by a later
# wait statement) depend on how this compiler allocates registers: another one may be
# fine, but only the parity tests and the resource report can say so.
CHECKED_HIPCC = "roc-7.2.0"


def check_compiler() -> None:
    """Refuses a compiler other than the checked one unless SONAR_ANY_HIPCC is set."""
    proc = subprocess.run([HIPCC, "--version"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if CHECKED_HIPCC in proc.stdout or os.environ.get("SONAR_ANY_HIPCC"):
        return
    raise RuntimeError(
        "%s is not the compiler these kernels were checked with (%s).  Set SONAR_ANY_HIPCC=1 to build "
        "anyway, then run tests/test_host_logic.py (no spills in the tile kernels) and the GPU parity "
        "tests before use.\n%s" % (HIPCC, CHECKED_HIPCC, proc.stdout))


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "unknown target feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_hip_library(verbose: bool = False, only=None) -> str:
    """Compiles every HIP source (or, with `only`, those sources; the other objects are
    reused when they exist) and links the shared library."""
    check_compiler()
    os.makedirs(LIB_DIR, exist_ok=True)
    only = set(only or HIP_SOURCES)

    def compile_one(src):
        obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
        if src in only or not os.path.exists(obj):
            cmd = [HIPCC, *HIP_FLAGS, "-I", os.path.join(ROOT, "include"), "-I", CSRC,
                   "-c", os.path.join(CSRC, src), "-o", obj]
            out = _run(cmd)
            if verbose and out.strip():
                print(out)
        return obj

    # one hipcc per source file, side by side
    with ThreadPoolExecutor(max_workers=min(len(HIP_SOURCES), os.cpu_count() or 1)) as pool:
        objs = list(pool.map(compile_one, HIP_SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    return LIB_PATH


def build_bench_library(verbose: bool = False) -> str:
    """Compiles the yardstick kernels bench.py times beside the GEMMs (an empty kernel, a
    kernel that only streams bytes) into a library of their own."""
    os.makedirs(LIB_DIR, exist_ok=True)
    out = _run([HIPCC, *HIP_FLAGS, "-shared", "-o", BENCH_PATH, os.path.join(CSRC, "bench_floor.hip")])
    if verbose and out.strip():
        print(out)
    return BENCH_PATH


def build_torch_ops(verbose: bool = False) -> str:
    """Compiles the C++ torch op registration layer with the host compiler and
    links it against the HIP library."""
    import torch
    from torch.utils import cpp_extension

    src = os.path.join(CSRC, "torch_bindings.cpp")
    inc = []
    for d in cpp_extension.include_paths():
        inc += ["-isystem", d]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi,
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-I", os.path.join(ROOT, "include"), "-isystem", "/opt/rocm/include", *inc, src,
           "-o", OPS_PATH, "-L", torch_lib, "-L", LIB_DIR,
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib,
           "-L", "/opt/rocm/lib", "-lsonar_marlin", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
           "-lamdhip64"]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return OPS_PATH


def build_all(verbose: bool = False):
    paths = [build_hip_library(verbose)]
    if os.path.exists(os.path.join(CSRC, "torch_bindings.cpp")):
        paths.append(build_torch_ops(verbose))
    paths.append(build_bench_library(verbose))
    return paths


if __name__ == "__main__":
    if len(sys.argv) > 1:   # python -m sonar_amd.build gemm_stream.hip ...: recompile these, relink
        print("built", build_hip_library(verbose=True, only=sys.argv[1:]))
    else:
        for p in build_all(verbose=True):
            print("built", p)
    sys.exit(0)
