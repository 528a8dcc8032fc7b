"""GPU parity at the full benchmark shapes (the inputs bench.py times).

The comparand is the reference itself - its own headers compiled into oracle/_ref/
libmshadow_ref.so, which travels with the tree - and, only where that library was not built,
the C restatement. Either finishes every operation at these sizes in well under a second on a
few cores, so each test compares the GPU result with it directly - bit for bit, except the
softmax forward (relative 1e-5: the device exponential is not libm's expf) - and then checks
a property that does not depend on any CPU implementation at all.
"""
import numpy as np
import pytest

import bench
from checkers import MAX, SAVETO, SUM, Checker, have_ref
from gpu_util import assert_bits_equal, f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import mshadow_amd
    g = mshadow_amd.load_cases()
    assert g.device_count() >= 1, "no GPU visible"
    g.set_device(0)
    return g


@pytest.fixture(scope="module")
def stream(G):
    s = G.stream_create()
    yield s
    G.stream_destroy(s)


@pytest.fixture(scope="module")
def O():
    return Checker("ref") if have_ref() else Checker("orc")


def test_the_comparand_is_the_compiled_reference_where_it_was_built(O):
    assert O.prefix == ("ref" if have_ref() else "orc")


@pytest.fixture(scope="module")
def H():
    return bench.make_inputs(1)


def test_map_fused_full(G, O, stream, H):
    want = np.empty_like(H["A"])
    O.map_fused(want, H["A"], H["B"], H["C"], H["D"])
    dev = [G.to_device(H[k]) for k in "ABCD"]
    out = G.buffer(H["A"].shape, f32)
    G.case_map_fused(out, *dev, 0, stream)
    got = out.download(stream)
    assert_bits_equal(got, want, "map 4096x4096")
    # sigmoid in (0,1), |A*B| <= 1, |D| <= 1
    assert np.all(got > -2.0) and np.all(got < 2.5)


def test_reductions_full(G, O, stream, H):
    x = H["X2a"]
    want = np.empty(256, f32)
    O.reduce_keep_highdim(want, x, SUM, SAVETO, 1.0)
    dst = G.buffer((256,), f32)
    src = G.to_device(x)
    G.reduce_keep_highdim(dst, src, SUM, SAVETO, 1.0, stream)
    got = dst.download(stream)
    assert_bits_equal(got, want, "sumall_except_dim<1> (64,256,56,56)")
    exact = x.astype(np.float64).sum(axis=(0, 2, 3))
    # a sequential fp32 sum of n unit-variance terms drifts by ~ sqrt(n) * eps * |partial sums|
    assert np.max(np.abs(got - exact)) < 0.05
    G.case_reduce_keep_highdim(dst, src, SUM, SAVETO, 1.0, 0, stream)
    assert_bits_equal(dst.download(stream), want, "sumall_except_dim<1> via expression")
    del src

    m = H["M2b"]
    want = np.empty(4096, f32)
    O.reduce_keep_lowest(want, m, SUM, SAVETO, 1.0)
    dst = G.buffer((4096,), f32)
    src = G.to_device(m)
    G.reduce_keep_lowest(dst, src, SUM, SAVETO, 1.0, stream)
    got = dst.download(stream)
    assert_bits_equal(got, want, "sum_rows 16384x4096")
    assert np.max(np.abs(got - m.astype(np.float64).sum(axis=0))) < 0.02
    G.case_reduce_keep_lowest(dst, src, SUM, SAVETO, 1.0, 0, stream)
    assert_bits_equal(dst.download(stream), want, "sum_rows via expression")
    G.reduce_keep_lowest(dst, src, MAX, SAVETO, 1.0, stream)
    assert_bits_equal(dst.download(stream), m.max(axis=0), "max over rows")


def test_softmax_and_grad_full(G, O, stream, H):
    x, lab = H["L"], H["labels"]
    want = np.empty_like(x)
    O.softmax(want, x)
    src = G.to_device(x)
    out = G.buffer(x.shape, f32)
    G.softmax(out, src, stream)
    got = out.download(stream)
    err = np.abs(got - want) / np.maximum(np.abs(want), np.finfo(f32).tiny)
    assert float(err.max()) <= 1e-5, float(err.max())
    rows = got.astype(np.float64).sum(axis=1)
    # the divisor is the sequential fp32 sum, which sits up to ~3e-5 below the exact one
    assert np.all(np.abs(rows - 1.0) < 5e-4)
    assert np.array_equal(got.argmax(axis=1), x.argmax(axis=1))
    del src
    # gradient of the GPU probabilities: bit-exact against the oracle on the same input
    wantg = np.empty_like(got)
    O.softmax_grad(wantg, got, lab)
    gout = G.buffer(x.shape, f32)
    G.softmax_grad(gout, out, G.to_device(lab), stream)
    gotg = gout.download(stream)
    assert_bits_equal(gotg, wantg, "softmax_grad 8192x32000")
    idx = lab.astype(np.int64)
    r = np.arange(x.shape[0])
    assert np.array_equal(gotg[r, idx], got[r, idx] - f32(1))
    gotg[r, idx] = got[r, idx]
    assert_bits_equal(gotg, got, "softmax_grad off-label entries")


def test_pool_unpool_full(G, O, stream, H):
    x, g = H["X4"], H["G4"]
    wantp = np.empty(g.shape, f32)
    O.pool(wantp, x, 3, 3, 2, 2, MAX)
    dx = G.to_device(x)
    dp = G.buffer(g.shape, f32)
    G.pool(dp, dx, 3, 3, 2, 2, MAX, stream)
    gotp = dp.download(stream)
    assert_bits_equal(gotp, wantp, "max pool (128,64,112,112)")
    # independent statement of the same windows through strided views
    win = np.lib.stride_tricks.sliding_window_view(x, (3, 3), axis=(2, 3))[:, :, ::2, ::2]
    assert_bits_equal(gotp, win.max(axis=(4, 5)), "max pool vs sliding windows")
    wantu = np.empty_like(x)
    O.unpool(wantu, x, wantp, g, 3, 3, 2, 2, MAX)
    du = G.buffer(x.shape, f32)
    G.unpool(du, dx, dp, G.to_device(g), 3, 3, 2, 2, MAX, stream)
    gotu = du.download(stream)
    assert_bits_equal(gotu, wantu, "max unpool (128,64,112,112)")
    # every window hands its gradient to each pixel that equals its maximum
    hits = (win == gotp[..., None, None]).sum(axis=(4, 5))
    tot = gotu.astype(np.float64).sum(axis=(2, 3))
    assert np.allclose(tot, (g.astype(np.float64) * hits).sum(axis=(2, 3)), rtol=0, atol=2e-2)


def test_im2col_col2im_full(G, O, stream):
    img, col = bench.half_inputs(1)
    n, c, h, w = img.shape
    wantc = np.empty(col.shape, np.uint16)
    O.im2col(wantc, img, 3, 3, 1, 1, 1, 1, 1, 1)
    dimg = G.to_device(img)
    dcol = G.buffer(col.shape, np.uint16)
    G.im2col(dcol, dimg, 3, 3, 1, 1, 1, 1, 1, 1, stream)
    gotc = dcol.download(stream)
    assert np.array_equal(gotc, wantc), "im2col f16 3x3 p1 (32,256,56,56)"
    # the centre tap (ky=1, kx=1) of every channel is the image itself
    centre = gotc.reshape(c, 3, 3, n, h, w)[:, 1, 1]
    assert np.array_equal(centre, img.transpose(1, 0, 2, 3))
    wanti = np.empty(img.shape, np.uint16)
    O.col2im(wanti, col, 3, 3, 1, 1, 1, 1, 1, 1)
    dout = G.buffer(img.shape, np.uint16)
    G.col2im(dout, G.to_device(col), 3, 3, 1, 1, 1, 1, 1, 1, stream)
    assert np.array_equal(dout.download(stream), wanti), "col2im f16"
    # col2im of im2col of an image of ones counts the windows covering each pixel
    ones = np.full(img.shape, 0x3C00, np.uint16)
    G.im2col(dcol, G.to_device(ones), 3, 3, 1, 1, 1, 1, 1, 1, stream)
    G.col2im(dout, dcol, 3, 3, 1, 1, 1, 1, 1, 1, stream)
    cnt = dout.download(stream).view(np.float16).astype(f32)
    ky = np.minimum(np.arange(h) + 1, 2) + np.minimum(h - 1 - np.arange(h), 1)
    kx = np.minimum(np.arange(w) + 1, 2) + np.minimum(w - 1 - np.arange(w), 1)
    assert np.array_equal(cnt, np.broadcast_to((ky[:, None] * kx[None, :]).astype(f32), cnt.shape))


@pytest.mark.gpu
@pytest.mark.parametrize("type_flag,dtype", [(3, np.uint8), (5, np.int8)])
def test_map_over_more_than_2_to_the_31_elements(G, stream, type_flag, dtype):
    """dst = a * b + c on 2^31 + 4096 one-byte elements (mshadow::kUint8 / kInt8): more than
    the 32-bit counters of one launch cover, so the view is evaluated in runs of rows and the
    leaves address it in 64 bits; checked against numpy's wrapping arithmetic"""
    rows, cols = 524289, 4096
    assert rows * cols == 2 ** 31 + 4096
    rng = np.random.default_rng(77)
    hosts = [rng.integers(0, 256, (rows, cols), dtype=np.uint8).view(dtype) for _ in range(3)]
    dev = [G.to_device(h, stream=stream) for h in hosts]
    dst = G.buffer((rows, cols), dtype)
    G.case_map_any(0, type_flag, dst, dev[0], dev[1], dev[2], stream)
    got = dst.download(stream)
    want = hosts[0] * hosts[1]
    want += hosts[2]
    assert np.array_equal(got, want)
    for d in dev + [dst]:
        d.free()
