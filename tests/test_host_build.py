"""CPU-only checks of what is built: exported C-ABI symbols, the host simulation of the
ordered sum, and the C++ header API evaluated on Tensor<cpu> against the oracle."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.path.join(ROOT, "mshadow_amd", "lib")


def _declared(header):
    path = os.path.join(ROOT, "include", header)
    if not os.path.exists(path):   # the probe library's header is no part of the boundary
        path = os.path.join(ROOT, "mshadow_amd", "csrc", header)
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b(mshadow_(?:hip|case|probe)_\w+)\s*\(", text)))


def _lib(name):
    path = os.path.join(LIBDIR, name)
    if not os.path.exists(path):
        import mshadow_amd.build as build

        build.build_all()
    # RTLD_LAZY is enough to resolve exports; nothing is called, so no GPU is needed
    return ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


@pytest.mark.parametrize("header,libname", [("mshadow_hip.h", "libmshadow_hip.so"),
                                            ("mshadow_hip_probe.h", "libmshadow_probe.so"),
                                            ("mshadow_hip_blas.h", "libmshadow_hip.so"),
                                            ("mshadow_hip_cases.h", "libmshadow_cases.so")])
def test_every_declared_symbol_is_exported(header, libname):
    names = _declared(header)
    assert len(names) >= (4 if "blas" in header or "probe" in header else 10)
    if libname == "libmshadow_cases.so":
        _lib("libmshadow_hip.so")
    lib = _lib(libname)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_fill_runs_of_rows_do_not_overflow():
    """tensor = scalar on 2^31 elements or more is launched in runs of whole rows; the run
    boundaries are host arithmetic and are checked here for shapes too large to allocate
    (INT_MAX rows of three elements: the row counter must not wrap)"""
    lib = _lib("libmshadow_hip.so")
    fn = lib.mshadow_hip_fill_32_runs
    fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int64), ctypes.c_int]
    for rows, cols, wide in ((2 ** 31 - 1, 3, 0), (2 ** 31 - 1, 2, 0), (2 ** 31 - 1, 8, 1), (70000, 65536, 1),
                             (5, 7, 0), (1, 2 ** 31 - 1, 0)):
        runs = (ctypes.c_int64 * 64)()
        n = fn(rows, cols, wide, runs, 32)
        assert 1 <= n <= 32, (rows, cols, n)
        units = cols // 4 if wide else cols
        at = 0
        for i in range(n):
            first, count = runs[2 * i], runs[2 * i + 1]
            assert first == at and count >= 1 and count * units < 2 ** 31, (rows, cols, i, first, count)
            at += count
        assert at == rows


def test_python_symbol_tables_match_headers():
    from mshadow_amd import capi

    assert sorted(capi.HIP_SYMBOLS) == sorted(_declared("mshadow_hip.h") +
                                              _declared("mshadow_hip_blas.h"))
    assert sorted(capi.CASES_SYMBOLS) == _declared("mshadow_hip_cases.h")


def test_expression_routes_reach_the_fixed_function_entries():
    """`dst = pool(...)`, `unpool`, `unpack_patch2col(pad(.))`, `crop(pack_col2patch(.))`,
    `transpose` / `swapaxis` of plain tensors and the reductions are recognised at compile
    time and handed to the library: the caller-style cases library, which only ever writes
    expressions, must therefore import those entry points"""
    if not os.path.exists(os.path.join(LIBDIR, "libmshadow_cases.so")):
        _lib("libmshadow_cases.so")
    out = subprocess.run(["nm", "-D", "--undefined-only", os.path.join(LIBDIR, "libmshadow_cases.so")],
                         check=True, capture_output=True, text=True).stdout
    imported = set(re.findall(r"\bU (mshadow_hip_\w+)", out))
    wanted = {"mshadow_hip_pool_f32", "mshadow_hip_unpool_f32", "mshadow_hip_im2col_f16",
              "mshadow_hip_im2col_f32", "mshadow_hip_col2im_f16", "mshadow_hip_col2im_f32",
              "mshadow_hip_permute_32", "mshadow_hip_reduce_keep_lowest_f32",
              "mshadow_hip_reduce_keep_highdim_f32", "mshadow_hip_softmax_f32",
              "mshadow_hip_sort_by_key_32", "mshadow_hip_blas_gemm", "mshadow_hip_blas_gemv",
              "mshadow_hip_blas_ger", "mshadow_hip_blas_dot"}
    assert wanted <= imported, sorted(wanted - imported)


def _symbols(path):
    out = subprocess.run(["readelf", "-Ws", "--wide", path], check=True, capture_output=True, text=True).stdout
    return [line.split()[-1] for line in out.splitlines() if " FUNC " in line or " OBJECT " in line]


@pytest.mark.parametrize("libname", ["libmshadow_hip.so", "libmshadow_cases.so"])
def test_host_and_device_halves_of_a_library_come_from_the_same_sources(libname, tmp_path):
    """hipcc compiles a file twice, once per side; a source edited between the two passes
    leaves launch stubs in the host code whose kernels are not in the gfx950 code object, and
    the first such launch ends the process. Every stub must find its kernel."""
    bundler = "/opt/rocm/llvm/bin/clang-offload-bundler"
    if not os.path.exists(bundler):
        pytest.skip("clang-offload-bundler not installed")
    _lib(libname)
    so = os.path.join(LIBDIR, libname)
    fat = str(tmp_path / "fat.bin")
    subprocess.run(["objcopy", "-O", "binary", "--only-section=.hip_fatbin", so, fat], check=True)
    # one bundle per source file of the library, back to back in the section
    magic = b"__CLANG_OFFLOAD_BUNDLE__"
    blob = open(fat, "rb").read()
    starts = [m.start() for m in re.finditer(re.escape(magic), blob)]
    assert starts, "no device code in " + libname
    kernels = set()
    for i, at in enumerate(starts):
        part, dev = str(tmp_path / f"bundle{i}.bin"), str(tmp_path / f"dev{i}.co")
        with open(part, "wb") as f:
            f.write(blob[at:starts[i + 1] if i + 1 < len(starts) else len(blob)])
        subprocess.run([bundler, "--unbundle", "--type=o", f"--input={part}", f"--output={dev}",
                        "--targets=hipv4-amdgcn-amd-amdhsa--gfx950"], check=True)
        kernels.update(_symbols(dev))

    def kernel_of(stub):
        # <len>__device_stub__<name> -> <len - 15><name>
        return re.sub(r"(\d+)__device_stub__", lambda m: str(int(m.group(1)) - 15), stub, count=1)
    stubs = [n for n in _symbols(so) if "__device_stub__" in n]
    assert len(stubs) > 100
    missing = [n for n in stubs if kernel_of(n) not in kernels]
    assert not missing, (len(missing), missing[:3])


def _compile_and_run(tmp_path, source, extra, args=()):
    exe = str(tmp_path / "check")
    cmd = ["g++", "-std=c++17", "-O2", "-fopenmp", "-ffp-contract=off", "-mf16c",
           "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "mshadow_amd"),
           "-o", exe, os.path.join(ROOT, "tests", "host", source)] + extra
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    out = subprocess.run([exe] + list(args), capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    return out.stdout


def test_ordered_sum_matches_serial_sum_on_host(tmp_path):
    """the lane arithmetic of the softmax row sum, driven lane by lane on the host,
    reproduces a strictly sequential float sum bit for bit"""
    out = _compile_and_run(tmp_path, "ordered_sum_sim.cc", [])
    assert out.startswith("OK"), out[-500:]


def test_planned_row_sum_matches_serial_sum_on_host(tmp_path):
    """the plan of the long-row softmax kernel (chunks and lanes classified from approximate
    prefix sums, a list of addends, every run verified) modelled on the host with the device
    code's own lane functions: bit-identical to a serial float sum wherever the plan holds,
    and it holds on every row shaped like a softmax's"""
    out = _compile_and_run(tmp_path, "row_plan_sim.cc", [])
    assert out.startswith("OK"), out[-500:]


def test_signed_column_sums_leave_most_of_the_chain(tmp_path):
    """sum_rows adds signed terms, and a plan of verified runs (what makes the softmax row sum
    parallel) leaves too much of its chain: cut with full knowledge of the true running sums,
    columns of 16384 N(0, 1) terms still keep 14 % of their dependent adds at a granularity of
    one term, 23 % at four (a lane's pack) and 70 % at 64 (a wave's load). The program rebuilds
    every column sum from its runs and compares it bit for bit with the serial loop."""
    out = _compile_and_run(tmp_path, "signed_plan_sim.cc", [], args=["48"])
    assert out.startswith("OK"), out[-500:]
    shares = {int(g): float(v) for g, v in re.findall(r"grain (\d+): ([0-9.]+)", out)}
    assert 0.10 < shares[1] < 0.18 and 0.18 < shares[4] < 0.30 and shares[64] > 0.6, shares


def test_half_sum_pruning_rule_is_exhaustively_sound(tmp_path):
    """the binary16 softmax row sum leaves out the terms below half an ulp of a lower bound of
    the running sum: for every pair of a finite non-negative binary16 sum and term the rule
    drops, half_t's `sum += term` indeed returns the sum unchanged (all 10^9 pairs)"""
    out = _compile_and_run(tmp_path, "half_prune_check.cc", [])
    assert out.startswith("OK"), out[-500:]
    dropped, kept_noops = (int(v) for v in out.split()[1:3])
    assert dropped > 10 ** 8 and kept_noops < 10 ** 5   # sound, and nearly tight (ties stay in)


def test_header_api_on_cpu_matches_oracle(tmp_path, orc):
    oracle_dir = os.path.join(ROOT, "oracle")
    out = _compile_and_run(tmp_path, "api_cpu_check.cc",
                           [os.path.join(oracle_dir, "liboracle.so"), "-Wl,-rpath," + oracle_dir])
    assert out.startswith("OK"), out


def test_half2_on_host_tensors(tmp_path):
    _lib("libmshadow_hip.so")
    out = _compile_and_run(tmp_path, "half2_check.cc",
                           ["-L" + LIBDIR, "-lmshadow_hip", "-Wl,-rpath," + LIBDIR])
    assert out.startswith("OK"), out


@pytest.mark.gpu
def test_half2_map_on_the_device():
    """x * x + x over half2_t elements: each lane is half_t arithmetic, rounded after the
    product and after the sum, which numpy's float16 does too"""
    import numpy as np
    import mshadow_amd
    G = mshadow_amd.load_cases()
    G.set_device(0)
    x = np.random.default_rng(8).uniform(-4, 4, 4096 + 6).astype(np.float16)
    want = (x * x).astype(np.float16) + x
    out = G.buffer(x.shape, np.uint16)
    G.case_half2_map(out, G.to_device(x.view(np.uint16)))
    assert np.array_equal(out.download(), want.astype(np.float16).view(np.uint16))


def _build_host_only_caller(tmp_path):
    exe = str(tmp_path / "hostonly")
    cmd = ["g++", "-std=c++17", "-O2", "-fopenmp", "-ffp-contract=off", "-mf16c",
           "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "mshadow_amd"),
           "-o", exe, os.path.join(ROOT, "tests", "host", "gpu_api_hostonly.cc"),
           "-L" + LIBDIR, "-lmshadow_hip", "-Wl,-rpath," + LIBDIR]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    return exe


def test_host_compiler_only_caller_builds(tmp_path):
    """Tensor<gpu> code whose assignments are all fixed-function operations needs no device
    compiler: g++ alone compiles it and links it against the library (run by a GPU test)"""
    _lib("libmshadow_hip.so")
    assert os.path.exists(_build_host_only_caller(tmp_path))


@pytest.mark.gpu
def test_host_compiler_only_caller_runs(tmp_path):
    out = subprocess.run([_build_host_only_caller(tmp_path)], capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0 and out.stdout.startswith("OK"), out.stdout[-2000:] + out.stderr[-2000:]
