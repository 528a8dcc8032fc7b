"""Matrix products: `dst <saver>= scale * dot(a[.T()], b[.T()])`, VectorDot, BatchGEMM, batch_dot.

One body (mshadow_amd/cases/dot_cases.inc) is compiled for Tensor<gpu>, for this backend's
Tensor<cpu> and - the three forms its stand-alone build knows - against the reference's headers.

Checker: the product in float64 (numpy). A BLAS is free to add in any order, so there is no
bit pattern to match; the bound used is 1e-5 of the largest magnitude of the result for inner
dimensions up to 512 (float accumulation gives about 1e-7 * sqrt(k)), 2e-3 for binary16
storage. The reference's own BLAS path (CBLAS / MKL on the host, cuBLAS on the device) cannot
be built in this image (no BLAS library), so parity with it is pinned by the mathematics and,
for the three forms it evaluates through implicit_dot, by the compiled reference.

Also here: the reference's own example and test programs (guide/basic.cpp, guide/defop.cpp,
test/test.cu, guide/basic_stream.cu), compiled unchanged against this backend's headers by
oracle/Makefile where the reference is present, are run and their output checked."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DROPIN = os.path.join(ROOT, "oracle", "_ref", "dropin")
f32 = np.float32
N_OPS = 17
DIMS = [(3, 4, 5, 2), (17, 33, 9, 3), (64, 128, 96, 4), (1, 1, 1, 1), (130, 257, 66, 2)]


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def operands(m, k, n, batch, seed=0):
    rng = np.random.default_rng(seed)
    size = batch * max(m * k, k * n, m * n) + 8
    return rng.standard_normal(size).astype(f32), rng.standard_normal(size).astype(f32)


def want_of(op, a, b, m, k, n, batch):
    """what op of dot_cases.inc must produce, in float64"""
    A, B = a.astype(np.float64), b.astype(np.float64)
    mk, kn = m * k, k * n
    if op == 0:
        return A[:mk].reshape(m, k) @ B[:kn].reshape(k, n)
    if op == 1:
        return A[:mk].reshape(m, k) @ B[:kn].reshape(n, k).T
    if op == 2:
        return A[:mk].reshape(k, m).T @ B[:kn].reshape(k, n)
    if op == 3:
        return A[:mk].reshape(k, m).T @ B[:kn].reshape(n, k).T
    if op == 4:
        return 1 + 0.5 * (A[:mk].reshape(m, k) @ B[:kn].reshape(k, n))
    if op == 5:
        return 1 - 2 * (A[:mk].reshape(m, k) @ B[:kn].reshape(n, k).T)
    if op == 6:
        return A[:k] @ B[:kn].reshape(k, n)
    if op == 7:
        return A[:k] @ B[:kn].reshape(n, k).T
    if op == 8:
        return np.outer(A[:m], B[:n])
    if op == 9:
        return 1 + 2 * np.outer(A[:m], B[:n])
    if op == 10:
        return np.array([A[:k] @ B[:k]])
    A3, B3 = A[:batch * mk], B[:batch * kn]
    if op == 11:
        return 1.5 * np.einsum("bmk,bkn->bmn", A3.reshape(batch, m, k), B3.reshape(batch, k, n))
    if op == 12:
        return 0.5 + np.einsum("bkm,bkn->bmn", A3.reshape(batch, k, m), B3.reshape(batch, k, n))
    if op == 13:
        return -np.einsum("bmk,bnk->bmn", A3.reshape(batch, m, k), B3.reshape(batch, n, k))
    if op == 14:
        return np.einsum("bmk,bkn->bmn", A3.reshape(batch, m, k), B3.reshape(batch, k, n))
    if op == 15:
        out = np.full((m, n + 5), -1.0)
        out[:, :n] = A[:mk].reshape(m, k) @ B[:kn].reshape(k, n)
        return out
    x, w = A[:mk].reshape(m, k), B[:kn].reshape(k, n)
    h = sigmoid(x @ w)
    return (h * (1 - h)) @ w.T


def close(got, want, what, tol=1e-5):
    got = np.asarray(got, np.float64).reshape(want.shape)
    assert np.all(np.isfinite(got)), what
    err = float(np.abs(got - want).max()) / max(1.0, float(np.abs(want).max()))
    assert err <= tol, (what, err)


def _ptr(x):
    return x.ctypes.data_as(ctypes.c_void_p)


# ----------------------------------------------------------------- host: Tensor<cpu>
@pytest.fixture(scope="module")
def host_lib(tmp_path_factory):
    so = str(tmp_path_factory.mktemp("hostdot") / "libhostcases.so")
    cmd = ["g++", "-std=c++17", "-O2", "-fopenmp", "-ffp-contract=off", "-mf16c", "-fPIC", "-shared",
           "-DDMLC_LOG_FATAL_THROW=1", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "mshadow_amd"), "-o", so,
           os.path.join(ROOT, "tests", "host", "ext_cpu_cases.cc")]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    lib = ctypes.CDLL(so)
    lib.host_dot_f32.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4
    return lib


@pytest.mark.parametrize("dims", DIMS)
@pytest.mark.parametrize("op", range(N_OPS))
def test_products_on_host_tensors(host_lib, op, dims):
    m, k, n, batch = dims
    a, b = operands(*dims, seed=op)
    want = want_of(op, a, b, *dims)
    out = np.full(want.size, np.nan, f32)
    assert host_lib.host_dot_f32(op, _ptr(out), _ptr(a), _ptr(b), m, k, n, batch) == 0
    close(out, want, f"host op {op} {dims}")


def test_unknown_case_is_an_error(host_lib):
    out, a = np.zeros(4, f32), np.zeros(4, f32)
    assert host_lib.host_dot_f32(99, _ptr(out), _ptr(a), _ptr(a), 1, 1, 1, 1) != 0


@pytest.mark.parametrize("dims", DIMS)
@pytest.mark.parametrize("op", range(3))
def test_products_of_the_compiled_reference(ref, host_lib, op, dims):
    """the forms the reference evaluates without an external BLAS agree with float64 and with
    this backend's host loops to the same bound"""
    m, k, n, batch = dims
    a, b = operands(*dims, seed=op)
    want = want_of(op, a, b, *dims)
    out = np.full(want.size, np.nan, f32)
    ref.dot(op, out, a, b, m, k, n)
    close(out, want, f"reference op {op} {dims}")
    mine = np.full(want.size, np.nan, f32)
    host_lib.host_dot_f32(op, _ptr(mine), _ptr(a), _ptr(b), m, k, n, 1)
    close(mine, out.astype(np.float64).reshape(want.shape), f"host vs reference op {op} {dims}")


# ----------------------------------------------------------------- a whole caller program
def two_layer_model(steps, eta, decay, x, label, w1, w2):
    """cases/two_layer_net.h in float64"""
    x, w1, w2 = x.astype(np.float64), w1.astype(np.float64), w2.astype(np.float64)
    batch = x.shape[0]
    b1, b2 = np.zeros(w1.shape[1]), np.zeros(w2.shape[1])
    onehot = np.zeros((batch, w2.shape[1]))
    onehot[np.arange(batch), label.astype(int)] = 1
    losses = []
    for _ in range(steps):
        act = sigmoid(x @ w1 + b1)
        z = act @ w2 + b2
        e = np.exp(z - z.max(axis=1, keepdims=True))
        p = e / e.sum(axis=1, keepdims=True)
        losses.append(float(-np.log(p[np.arange(batch), label.astype(int)]).mean()))
        g = (p - onehot) / batch
        gb2, gw2 = g.sum(axis=0), act.T @ g
        ga = act * (1 - act) * (g @ w2.T)
        gb1, gw1 = ga.sum(axis=0), x.T @ ga
        w1 -= eta * (decay * w1 + gw1)
        w2 -= eta * (decay * w2 + gw2)
        b1 -= eta * gb1
        b2 -= eta * gb2
    return w1, w2, p, losses


def two_layer_problem():
    rng = np.random.default_rng(21)
    batch, n_in, n_hidden, n_out = 96, 50, 40, 10
    centres = rng.standard_normal((n_out, n_in))
    label = rng.integers(0, n_out, batch)
    x = (centres[label] + 0.3 * rng.standard_normal((batch, n_in))).astype(f32)
    w1 = (0.1 * rng.standard_normal((n_in, n_hidden))).astype(f32)
    w2 = (0.1 * rng.standard_normal((n_hidden, n_out))).astype(f32)
    return x, label.astype(f32), w1, w2


def check_two_layer(run, what):
    steps, eta, decay = 30, 0.8, 1e-5
    x, label, w1, w2 = two_layer_problem()
    mw1, mw2, mp, losses = two_layer_model(steps, eta, decay, x, label, w1, w2)
    assert losses[-1] < 0.5 * losses[0], "the model problem does not train"
    probs = np.full(mp.shape, np.nan, f32)
    run(steps, eta, decay, x, label, w1, w2, probs)
    close(w1, mw1, what + " w1", 1e-4)
    close(w2, mw2, what + " w2", 1e-4)
    close(probs, mp, what + " probabilities", 1e-4)


def test_two_layer_net_on_the_host(host_lib):
    fl, ip = ctypes.c_float, ctypes.c_int
    host_lib.host_two_layer_net_f32.argtypes = [ip, fl, fl, ip, ip, ip, ip] + [ctypes.c_void_p] * 5

    def run(steps, eta, decay, x, label, w1, w2, probs):
        assert host_lib.host_two_layer_net_f32(steps, eta, decay, x.shape[0], x.shape[1], w1.shape[1],
                                               w2.shape[1], _ptr(x), _ptr(label), _ptr(w1), _ptr(w2),
                                               _ptr(probs)) == 0
    check_two_layer(run, "host")


# ----------------------------------------------------------------- the reference's own programs, host
def _run(name, *args):
    exe = os.path.join(DROPIN, name)
    if not os.path.exists(exe):
        pytest.skip(f"{exe} not built (oracle/Makefile builds it where /root/reference is present)")
    return subprocess.run([exe] + list(args), capture_output=True, text=True, timeout=120)


def test_guide_defop_prints_what_the_reference_prints():
    mine, theirs = _run("defop"), _run("defop_reference")
    assert mine.returncode == 0 and theirs.returncode == 0
    assert mine.stdout == theirs.stdout and len(mine.stdout) > 0


def test_guide_basic_runs_to_the_end():
    """guide/basic.cpp reaches VectorDot after its first two blocks of output; the reference's
    stand-alone build stops there (its BLAS-less engine has no vector product), this backend
    carries on. Up to that point the two must print the same text; after it the program's own
    checks are arithmetic on small integers, compared here with what they must give."""
    mine, theirs = _run("basic"), _run("basic_reference")
    assert mine.returncode == 0, mine.stderr[-2000:]
    head = theirs.stdout
    assert len(head) > 20 and mine.stdout.startswith(head)
    rest = mine.stdout[len(head):]
    assert rest.startswith("vdot=3.000000\n3.00 3.00 \n3.00 3.00 \n")
    lines = mine.stdout.splitlines()
    # pool<red::sum> with a 3x3 window and stride 3 over the 3x nearest upsampling of [[1,2],[3,4]]
    at = lines.index("upsampling")
    assert lines[at + 1:at + 9] == ["1.00 1.00 1.00 2.00 2.00 2.00 "] * 3 + \
        ["3.00 3.00 3.00 4.00 4.00 4.00 "] * 3 + ["9.00 18.00 ", "27.00 36.00 "]


# ----------------------------------------------------------------- device
@pytest.fixture(scope="module")
def G():
    import mshadow_amd
    g = mshadow_amd.load_cases()
    assert g.device_count() >= 1, "no GPU visible"
    g.set_device(0)
    return g


@pytest.mark.gpu
@pytest.mark.parametrize("dims", DIMS + [(512, 512, 384, 3)])
@pytest.mark.parametrize("op", range(N_OPS))
def test_products_on_device_tensors(G, op, dims):
    m, k, n, batch = dims
    a, b = operands(*dims, seed=op)
    want = want_of(op, a, b, *dims)
    s = G.stream_create()
    out = G.buffer((want.size,), f32)
    G.case_dot(op, out, G.to_device(a), G.to_device(b), m, k, n, batch, s)
    close(out.download(s), want, f"device op {op} {dims}")


@pytest.mark.gpu
def test_unknown_case_is_an_error_on_the_device_too(G):
    from mshadow_amd.capi import HipError
    buf = G.buffer((4,), f32)
    with pytest.raises(HipError):
        G.case_dot(99, buf, buf, buf, 1, 1, 1)


@pytest.mark.gpu
def test_two_layer_net_on_the_device(G):
    """Copy in, 30 updates of dot / repmat / F<> / Softmax / SoftmaxGrad / sum_rows / scaled
    saves on one stream, Copy out: the float64 model's weights and probabilities to 1e-4"""
    s = G.stream_create()
    check_two_layer(lambda *a: G.case_two_layer_net(*a, stream=s), "device")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_name", ["f32", "f64", "f16"])
@pytest.mark.parametrize("transa,transb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_abi_gemm(G, dtype_name, transa, transb):
    """mshadow_hip_blas_gemm: leading dimensions larger than the rows, alpha / beta, a batch
    by stride"""
    from mshadow_amd import capi
    code, dt, tol = {"f32": (capi.BLAS_F32, np.float32, 1e-5), "f64": (capi.BLAS_F64, np.float64, 1e-12),
                     "f16": (capi.BLAS_F16, np.float16, 2e-3)}[dtype_name]
    rng = np.random.default_rng(3)
    m, n, k, batch = 37, 29, 53, 3
    ar, ac = (k, m) if transa else (m, k)
    br, bc = (n, k) if transb else (k, n)
    lda, ldb, ldc = ar + 3, br + 1, m + 2
    A = np.zeros((batch, ac, lda), dt)   # column-major with padding rows: [batch][col][row]
    B = np.zeros((batch, bc, ldb), dt)
    Cm = np.zeros((batch, n, ldc), dt)
    A[:, :, :ar] = rng.standard_normal((batch, ac, ar))
    B[:, :, :br] = rng.standard_normal((batch, bc, br))
    Cm[:, :, :m] = rng.standard_normal((batch, n, m))
    Cm[:, :, m:] = 7.0
    alpha, beta = 0.75, -0.5
    opA = (A[:, :, :ar].astype(np.float64).transpose(0, 2, 1))   # (batch, ar, ac) = stored matrix
    opB = (B[:, :, :br].astype(np.float64).transpose(0, 2, 1))
    if transa:
        opA = opA.transpose(0, 2, 1)
    if transb:
        opB = opB.transpose(0, 2, 1)
    C0 = Cm[:, :, :m].astype(np.float64).transpose(0, 2, 1)
    want = alpha * opA @ opB + beta * C0
    dA, dB, dC = G.to_device(A.reshape(-1)), G.to_device(B.reshape(-1)), G.to_device(Cm.reshape(-1))
    s = G.stream_create()
    G.blas_gemm(code, transa, transb, m, n, k, alpha, dA, lda, dB, ldb, beta, dC, ldc, batch,
                (ac * lda, bc * ldb, n * ldc), s)
    got = dC.download(s).reshape(batch, n, ldc)
    assert np.all(got[:, :, m:] == 7.0), "padding rows of C were written"
    close(got[:, :, :m].transpose(0, 2, 1), want, f"gemm {dtype_name} {transa}{transb}", tol)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_name", ["f32", "f64"])
def test_abi_gemv_ger_dot(G, dtype_name):
    from mshadow_amd import capi
    code, dt, tol = {"f32": (capi.BLAS_F32, np.float32, 1e-5),
                     "f64": (capi.BLAS_F64, np.float64, 1e-12)}[dtype_name]
    rng = np.random.default_rng(4)
    m, n, lda = 45, 31, 48
    A = np.zeros((n, lda), dt)
    A[:, :m] = rng.standard_normal((n, m))
    Am = A[:, :m].astype(np.float64).T            # the m x n matrix
    s = G.stream_create()
    for trans in (0, 1):
        xlen, ylen = (m, n) if trans else (n, m)
        x = rng.standard_normal(xlen * 2).astype(dt)     # incx = 2
        y = rng.standard_normal(ylen).astype(dt)
        want = 1.25 * (Am.T if trans else Am) @ x[::2].astype(np.float64) + 0.5 * y
        dy = G.to_device(y)
        G.blas_gemv(code, trans, m, n, 1.25, G.to_device(A.reshape(-1)), lda, G.to_device(x), 2, 0.5,
                    dy, 1, stream=s)
        close(dy.download(s), want, f"gemv {dtype_name} trans={trans}", tol)
    x = rng.standard_normal(m).astype(dt)
    y = rng.standard_normal(n).astype(dt)
    dA = G.to_device(A.reshape(-1))
    G.blas_ger(code, m, n, -2.0, G.to_device(x), 1, G.to_device(y), 1, dA, lda, stream=s)
    got = dA.download(s).reshape(n, lda)
    assert np.all(got[:, m:] == 0), "padding rows of A were written"
    close(got[:, :m].T, Am - 2.0 * np.outer(x.astype(np.float64), y.astype(np.float64)),
          f"ger {dtype_name}", tol)
    u = rng.standard_normal(10001).astype(dt)
    v = rng.standard_normal(10001).astype(dt)
    res = G.buffer((1,), dt)
    G.blas_dot(code, 10001, G.to_device(u), 1, G.to_device(v), 1, res, s)
    close(res.download(s), np.array([u.astype(np.float64) @ v.astype(np.float64)]),
          f"dot {dtype_name}", tol * 100)   # relative to max(1, |result|): cancellation in the sum


@pytest.mark.gpu
def test_abi_rejects_what_would_read_out_of_bounds(G):
    from mshadow_amd import capi
    from mshadow_amd.capi import HipError
    buf = G.buffer((64,), f32)
    with pytest.raises(HipError, match="lda"):
        G.blas_gemm(capi.BLAS_F32, 0, 0, 8, 8, 8, 1.0, buf, 4, buf, 8, 0.0, buf, 8)
    with pytest.raises(HipError, match="ldc"):
        G.blas_gemm(capi.BLAS_F32, 0, 0, 8, 8, 8, 1.0, buf, 8, buf, 8, 0.0, buf, 7)
    with pytest.raises(HipError, match="overlap"):
        G.blas_gemm(capi.BLAS_F32, 0, 0, 2, 2, 2, 1.0, buf, 2, buf, 2, 0.0, buf, 2, 4, (4, 4, 2))
    with pytest.raises(HipError, match="element type"):
        G.blas_gemm(7, 0, 0, 2, 2, 2, 1.0, buf, 2, buf, 2, 0.0, buf, 2)
    with pytest.raises(HipError, match="float and double"):
        G.blas_gemv(capi.BLAS_F16, 0, 2, 2, 1.0, buf, 2, buf, 1, 0.0, buf, 1)
    with pytest.raises(HipError, match="increment"):
        G.blas_ger(capi.BLAS_F32, 2, 2, 1.0, buf, 0, buf, 1, buf, 2)
    # empty problems are accepted and do nothing
    G.blas_gemm(capi.BLAS_F32, 0, 0, 0, 8, 8, 1.0, buf, 1, buf, 8, 0.0, buf, 1)
    # an empty inner dimension leaves beta * C, as BLAS defines it
    c = G.to_device(np.arange(6, dtype=f32))
    G.blas_gemm(capi.BLAS_F32, 0, 0, 2, 3, 0, 1.0, buf, 2, buf, 1, 0.5, c, 2)
    assert np.array_equal(c.download(), np.arange(6, dtype=f32) * f32(0.5))


# ----------------------------------------------------------------- the reference's own programs, device
@pytest.mark.gpu
def test_reference_test_cu_passes_on_this_backend():
    """test/test.cu of the reference, unchanged: copies, sum_rows, sumall_except_dim<0>, Softmax
    and mirror on Tensor<gpu> against Tensor<cpu>; it asserts agreement itself and prints one
    confirmation per block"""
    out = _run("test_cu")
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    assert out.stdout.count("cpu & gpu result consists") == 4
    assert "batch 1 of gpu & cpu tensor are same." in out.stdout
    lines = out.stdout.splitlines()
    # sum_rows of tc[0] = [[0,.1,.2,.3],[.2,.3,.4,.5]] and its copy from the device
    at = lines.index("#sum_rows of batch 0:")
    assert lines[at + 1] == "0.20 0.40 0.60 0.80 " and lines[at + 3] == "0.20 0.40 0.60 0.80 "


@pytest.mark.gpu
def test_reference_basic_stream_cu_multiplies_on_three_streams():
    """guide/basic_stream.cu of the reference, unchanged: two fills on two streams and a
    product on a third; (2x5 of ones) x (2x5 of twos)^T = 10 everywhere"""
    out = _run("basic_stream_cu")
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    assert out.stdout == "10.00 10.00 \n10.00 10.00 \n"
