"""The hot path as one program: the convolutional network of cases/conv_net.h (the network of the
reference's guide/neuralnet/convnet.cu with today's signatures) compiled for Tensor<gpu>, for
this backend's Tensor<cpu> and against the reference's own headers, compared tensor by tensor.

Two kinds of run:
  * exact: inputs, weights and the gradient that enters the backward pass are small dyadic
    numbers, chosen so that every matrix product and every sum in the chain is exact in
    float32 whatever the order of its additions. Then the three builds must agree BIT FOR BIT on
    every tensor of the chain (patch matrix, convolution, activations, pooling, logits, all
    gradients, the updated weights) - the library products included - except the softmax
    probabilities, whose exponential comes from different libraries (relative 1e-5).
  * trained: ordinary float data, several rounds; the matrix products now differ in the order of
    their additions, so tensors agree to 1e-4 of their largest magnitude.
"""
import ctypes
import os
import subprocess

import numpy as np
import pytest

from checkers import REF_SO, have_ref
from gpu_util import assert_bits_equal, f32

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

KEPT = ("col_forward", "conv_raw", "hidden", "pooled", "logits", "probs", "grad_out_bias",
        "grad_out_weight", "flat_grad", "unpooled", "hidden_grad", "grad_hidden_bias", "grad_kernel",
        "col_backward", "input_grad", "hidden_bias", "out_bias")


class Geometry:
    def __init__(self, batch, in_channels, in_size, channels, ksize, kstride, pad, psize, num_out):
        self.v = (batch, in_channels, in_size, channels, ksize, kstride, pad, psize, num_out)
        (self.batch, self.in_channels, self.in_size, self.channels, self.ksize, self.kstride, self.pad,
         self.psize, self.num_out) = self.v
        self.conv_out = (in_size + 2 * pad - ksize) // kstride + 1
        self.pool_out = (self.conv_out + 1 - psize) // psize
        self.flat = channels * self.pool_out ** 2
        self.patch = in_channels * ksize * ksize
        self.positions = batch * self.conv_out ** 2

    def array(self):
        return (ctypes.c_int * 9)(*self.v)

    def shapes(self):
        b, c, co, po = self.batch, self.channels, self.conv_out, self.pool_out
        hidden = (b, c, co, co)
        return {"col_forward": (self.patch, self.positions), "col_backward": (self.patch, self.positions),
                "conv_raw": (c, self.positions), "hidden": hidden, "unpooled": hidden, "hidden_grad": hidden,
                "pooled": (b, c, po, po), "flat_grad": (b, self.flat), "logits": (b, self.num_out),
                "probs": (b, self.num_out), "grad_out_bias": (self.num_out,), "out_bias": (self.num_out,),
                "grad_out_weight": (self.flat, self.num_out), "grad_hidden_bias": (c,), "hidden_bias": (c,),
                "grad_kernel": (c, self.patch), "input_grad": (b, self.in_channels, self.in_size, self.in_size)}


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def run_net(fn, g, steps, eta, decay, images, labels, fixed_grad, kernel, weight, stream=False):
    """-> (dict of kept tensors, trained kernel, trained weight)"""
    shapes = g.shapes()
    kept = {k: np.full(shapes[k], np.nan, f32) for k in KEPT}
    keep = (ctypes.c_void_p * len(KEPT))(*[kept[k].ctypes.data for k in KEPT])
    kernel, weight = kernel.copy(), weight.copy()
    args = [g.array(), steps, ctypes.c_float(eta), ctypes.c_float(decay), _p(images), _p(labels),
            _p(fixed_grad), _p(kernel), _p(weight), keep]
    if stream is not False:
        args.append(stream)
    status = fn(*args)
    assert status in (0, None), status
    return kept, kernel, weight


@pytest.fixture(scope="module")
def host_lib(tmp_path_factory):
    so = str(tmp_path_factory.mktemp("hostconv") / "libhostcases.so")
    cmd = ["g++", "-std=c++17", "-O2", "-fopenmp", "-ffp-contract=off", "-mf16c", "-fPIC", "-shared",
           "-DDMLC_LOG_FATAL_THROW=1", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "mshadow_amd"), "-o", so,
           os.path.join(ROOT, "tests", "host", "ext_cpu_cases.cc")]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    lib = ctypes.CDLL(so)
    lib.host_conv_net_f32.restype = ctypes.c_int
    lib.host_conv_pair.restype = ctypes.c_int
    return lib


@pytest.fixture(scope="module")
def ref_lib():
    if not have_ref():
        pytest.skip("oracle/_ref/libmshadow_ref.so not built (needs /root/reference)")
    lib = ctypes.CDLL(REF_SO)
    lib.ref_conv_net_f32.restype = None
    lib.ref_conv_pair.restype = None
    return lib


def dyadic_case(g, seed):
    """inputs for which every product and sum of one round is exact in float32 (pixels in
    {0..3}/4, weights in {-2..2}/4, the entering gradient in {-4..4}/16; the sums stay far
    below 2^24 units of their grid), and an update with power-of-two rates"""
    rng = np.random.default_rng(seed)
    images = (rng.integers(0, 4, (g.batch, g.in_channels, g.in_size, g.in_size)) / 4).astype(f32)
    kernel = (rng.integers(-2, 3, (g.channels, g.patch)) / 4).astype(f32)
    weight = (rng.integers(-2, 3, (g.flat, g.num_out)) / 4).astype(f32)
    grad = (rng.integers(-4, 5, (g.batch, g.num_out)) / 16).astype(f32)
    labels = rng.integers(0, g.num_out, g.batch).astype(f32)
    return images, labels, grad, kernel, weight


GEOMETRIES = [Geometry(8, 1, 28, 10, 5, 1, 0, 2, 10),     # the reference program's own sizes, a small batch
              Geometry(4, 3, 16, 8, 3, 1, 1, 2, 6),       # several input channels, a padded 3x3 convolution
              Geometry(3, 2, 17, 5, 4, 2, 0, 3, 7)]       # stride 2, windows of 3, odd sizes


def compare_exact(got, want, g, what):
    for k in KEPT:
        if k == "probs":
            rel = np.abs(got[k].astype(np.float64) - want[k]) / want[k]
            assert rel.max() <= 1e-5, (what, k, rel.max())
        else:
            assert_bits_equal(got[k], want[k], f"{what}: {k}")


@pytest.mark.parametrize("gi", range(len(GEOMETRIES)))
def test_cpu_device_equals_reference_bit_for_bit(host_lib, ref_lib, gi):
    """this backend's Tensor<cpu> against the reference's: same loops, same libm, so every
    tensor of the chain is identical, the probabilities too - on dyadic and on ordinary data"""
    g = GEOMETRIES[gi]
    images, labels, grad, kernel, weight = dyadic_case(g, 100 + gi)
    a = run_net(host_lib.host_conv_net_f32, g, 1, 0.125, 2.0 ** -6, images, labels, grad, kernel, weight)
    b = run_net(ref_lib.ref_conv_net_f32, g, 1, 0.125, 2.0 ** -6, images, labels, grad, kernel, weight)
    for k in KEPT:
        assert_bits_equal(a[0][k], b[0][k], k)
    assert_bits_equal(a[1], b[1], "kernel")
    assert_bits_equal(a[2], b[2], "weight")
    rng = np.random.default_rng(gi)
    images = rng.standard_normal(images.shape, dtype=f32)
    kernel = rng.standard_normal(kernel.shape, dtype=f32) * f32(0.1)
    weight = rng.standard_normal(weight.shape, dtype=f32) * f32(0.1)
    a = run_net(host_lib.host_conv_net_f32, g, 3, 0.1, 1e-5, images, labels, None, kernel, weight)
    b = run_net(ref_lib.ref_conv_net_f32, g, 3, 0.1, 1e-5, images, labels, None, kernel, weight)
    for k in KEPT:
        assert_bits_equal(a[0][k], b[0][k], k)
    assert_bits_equal(a[1], b[1], "kernel")


def test_exact_case_is_exact_in_any_order(ref_lib):
    """what makes the GPU comparison below meaningful: on the dyadic inputs the reference's
    result does not depend on the order of the additions - a float64 evaluation of the
    convolution, the logits and the kernel gradient gives the same numbers"""
    g = GEOMETRIES[1]
    images, labels, grad, kernel, weight = dyadic_case(g, 101)
    kept, _, _ = run_net(ref_lib.ref_conv_net_f32, g, 1, 0.125, 2.0 ** -6, images, labels, grad, kernel, weight)
    conv = kernel.astype(np.float64) @ kept["col_forward"].astype(np.float64)
    assert np.array_equal(conv, kept["conv_raw"].astype(np.float64))
    flat = kept["pooled"].reshape(g.batch, -1).astype(np.float64)
    assert np.array_equal(flat @ weight.astype(np.float64), kept["logits"].astype(np.float64))
    swapped = kept["hidden_grad"].transpose(1, 0, 2, 3).reshape(g.channels, -1).astype(np.float64)
    assert np.array_equal(swapped @ kept["col_forward"].astype(np.float64).T,
                          kept["grad_kernel"].astype(np.float64))
    # and the probabilities are a softmax of the logits
    e = np.exp(kept["logits"].astype(np.float64) - kept["logits"].max(axis=1, keepdims=True))
    assert np.allclose(kept["probs"], e / e.sum(axis=1, keepdims=True), rtol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("gi", range(len(GEOMETRIES)))
def test_gpu_chain_equals_reference_bit_for_bit_on_exact_inputs(ref_lib, gi):
    import mshadow_amd
    G = mshadow_amd.load_cases()
    G.set_device(0)
    stream = G.stream_create()
    g = GEOMETRIES[gi]
    images, labels, grad, kernel, weight = dyadic_case(g, 100 + gi)
    want = run_net(ref_lib.ref_conv_net_f32, g, 1, 0.125, 2.0 ** -6, images, labels, grad, kernel, weight)
    fn = G.cases.mshadow_case_conv_net_f32
    got = run_net(fn, g, 1, 0.125, 2.0 ** -6, images, labels, grad, kernel, weight, stream=stream)
    compare_exact(got[0], want[0], g, f"geometry {g.v}")
    assert_bits_equal(got[1], want[1], "kernel after the update")
    assert_bits_equal(got[2], want[2], "weight after the update")
    G.stream_destroy(stream)


@pytest.mark.gpu
@pytest.mark.parametrize("gi", range(len(GEOMETRIES)))
def test_gpu_training_rounds_agree_with_reference(ref_lib, gi):
    import mshadow_amd
    G = mshadow_amd.load_cases()
    G.set_device(0)
    stream = G.stream_create()
    g = GEOMETRIES[gi]
    rng = np.random.default_rng(7 + gi)
    images = rng.standard_normal((g.batch, g.in_channels, g.in_size, g.in_size), dtype=f32)
    kernel = rng.standard_normal((g.channels, g.patch), dtype=f32) * f32(0.1)
    weight = rng.standard_normal((g.flat, g.num_out), dtype=f32) * f32(0.1)
    labels = rng.integers(0, g.num_out, g.batch).astype(f32)
    want = run_net(ref_lib.ref_conv_net_f32, g, 4, 0.1, 1e-5, images, labels, None, kernel, weight)
    got = run_net(G.cases.mshadow_case_conv_net_f32, g, 4, 0.1, 1e-5, images, labels, None, kernel, weight,
                  stream=stream)
    for k in KEPT + ("kernel", "weight"):
        a = got[0][k] if k in got[0] else got[1 if k == "kernel" else 2]
        b = want[0][k] if k in want[0] else want[1 if k == "kernel" else 2]
        scale = max(float(np.abs(b).max()), 1e-30)
        err = float(np.abs(a.astype(np.float64) - b).max()) / scale
        assert err <= 1e-4, (k, err)
    G.stream_destroy(stream)


PAIR_GEOMETRIES = [Geometry(2, 4, 56, 8, 3, 1, 1, 2, 1),   # 3x3, stride 1, pad 1, rows of whole packs
                   Geometry(3, 2, 13, 5, 3, 2, 0, 2, 1),   # the general patch kernels
                   Geometry(2, 3, 20, 4, 5, 1, 2, 2, 1)]


def pair_case(g, seed, half):
    rng = np.random.default_rng(seed)
    image = (rng.integers(0, 4, (g.batch, g.in_channels, g.in_size, g.in_size)) / 4).astype(f32)
    kernel = (rng.integers(-2, 3, (g.channels, g.patch)) / 4).astype(f32)
    grad = (rng.integers(-2, 3, (g.batch, g.channels, g.conv_out, g.conv_out)) / 4).astype(f32)
    if half:
        return [a.astype(np.float16).view(np.uint16) for a in (image, kernel, grad)]
    return [image, kernel, grad]


def run_pair(fn, g, half, operands, stream=False):
    dt = np.uint16 if half else f32
    outs = [np.zeros((g.patch, g.positions), dt), np.zeros((g.batch, g.channels, g.conv_out, g.conv_out), dt),
            np.zeros((g.patch, g.positions), dt), np.zeros((g.batch, g.in_channels, g.in_size, g.in_size), dt)]
    args = [int(half), g.array()] + [_p(a) for a in operands] + [_p(a) for a in outs]
    if stream is not False:
        args.append(stream)
    assert fn(*args) in (0, None)
    return outs


@pytest.mark.parametrize("half", [0, 1])
@pytest.mark.parametrize("gi", range(len(PAIR_GEOMETRIES)))
def test_convolution_pair_cpu_device_equals_reference(host_lib, ref_lib, gi, half):
    g = PAIR_GEOMETRIES[gi]
    ops = pair_case(g, 40 + gi, half)
    a = run_pair(host_lib.host_conv_pair, g, half, ops)
    b = run_pair(ref_lib.ref_conv_pair, g, half, ops)
    for x, y, name in zip(a, b, ("col_forward", "out", "col_backward", "image_grad")):
        assert_bits_equal(x, y, name)
    # the convolution against a direct float64 evaluation (exact on these inputs)
    img, ker = (ops[0].view(np.float16) if half else ops[0]), (ops[1].view(np.float16) if half else ops[1])
    padded = np.pad(img.astype(np.float64), ((0, 0), (0, 0), (g.pad, g.pad), (g.pad, g.pad)))
    want = np.zeros((g.batch, g.channels, g.conv_out, g.conv_out))
    k4 = ker.astype(np.float64).reshape(g.channels, g.in_channels, g.ksize, g.ksize)
    for oy in range(g.conv_out):
        for ox in range(g.conv_out):
            win = padded[:, :, oy * g.kstride: oy * g.kstride + g.ksize, ox * g.kstride: ox * g.kstride + g.ksize]
            want[:, :, oy, ox] = np.einsum("bcyx,kcyx->bk", win, k4)
    out = b[1].view(np.float16) if half else b[1]
    assert np.array_equal(out.astype(np.float64), want)


@pytest.mark.gpu
@pytest.mark.parametrize("half", [0, 1])
@pytest.mark.parametrize("gi", range(len(PAIR_GEOMETRIES)))
def test_gpu_convolution_pair_equals_reference_bit_for_bit(ref_lib, gi, half):
    import mshadow_amd
    G = mshadow_amd.load_cases()
    G.set_device(0)
    stream = G.stream_create()
    g = PAIR_GEOMETRIES[gi]
    ops = pair_case(g, 40 + gi, half)
    want = run_pair(ref_lib.ref_conv_pair, g, half, ops)
    got = run_pair(G.cases.mshadow_case_conv_pair, g, half, ops, stream=stream)
    for x, y, name in zip(got, want, ("col_forward", "out", "col_backward", "image_grad")):
        assert_bits_equal(x, y, f"{name} {g.v} half={half}")
    G.stream_destroy(stream)
