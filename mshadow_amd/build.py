"""Build recipe for the native parts (gfx950 only).

  libmshadow_hip.so    the C ABI device layer (csrc/runtime.hip, csrc/ops.hip, csrc/sort.hip,
                       csrc/permute.hip, csrc/random.hip)
  libmshadow_cases.so  caller-style programs written against <mshadow/tensor.h>
                       (cases/cases.hip), exported as C functions for tests and bench
  libmshadow_probe.so  measurement aids of bench.py (csrc/probe.hip); nothing depends on it

Both are built in-tree under mshadow_amd/lib/ with hipcc, which cross-compiles without a
GPU. Flags that matter for results:
  -ffp-contract=off                 a*b+c stays a multiply and an add, like the CPU path
  -target-feature -packed-fp32-ops  no packed-FP32 instructions
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_DIR = os.path.join(HERE, "lib")
HIP_SO = os.path.join(LIB_DIR, "libmshadow_hip.so")
CASES_SO = os.path.join(LIB_DIR, "libmshadow_cases.so")
PROBE_SO = os.path.join(LIB_DIR, "libmshadow_probe.so")

ARCH = "gfx950"
COMMON = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    f"-I{os.path.join(ROOT, 'include')}", f"-I{HERE}",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _run(cmd, verbose):
    if verbose:
        print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"build failed ({res.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)


def build_hip_library(verbose=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = [os.path.join(HERE, "csrc", f) for f in ("runtime.hip", "ops.hip", "sort.hip", "permute.hip", "random.hip", "blas.hip")]
    # -ldl: blas.hip opens rocBLAS at run time, on the first matrix product
    _run([hipcc()] + COMMON + ["-o", HIP_SO] + srcs + ["-ldl"], verbose)
    return HIP_SO


def build_cases_library(verbose=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(HERE, "cases", "cases.hip")
    _run([hipcc()] + COMMON + ["-o", CASES_SO, src, f"-L{LIB_DIR}", "-lmshadow_hip",
                               "-Wl,-rpath,$ORIGIN"], verbose)
    return CASES_SO


def build_probe_library(verbose=True):
    """measurement aids for bench.py: instrumented copies of library kernels, micro-benchmarks"""
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(HERE, "csrc", "probe.hip")
    _run([hipcc()] + COMMON + ["-o", PROBE_SO, src], verbose)
    return PROBE_SO


def build_all(verbose=True):
    build_hip_library(verbose)
    build_cases_library(verbose)
    build_probe_library(verbose)


if __name__ == "__main__":
    build_all("-q" not in sys.argv)
