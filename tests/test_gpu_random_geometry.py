"""GPU parity on seeded random shapes: pool / unpool, patch2col / col2patch, Softmax and its
gradient, the two reductions.

The hand-picked cases of test_gpu_parity.py sit on the borders the kernels' dispatch knows of;
these draw window, stride, padding, sizes and pitch at random (fixed seeds, so a failure names
its case), with a bias towards the sizes where the routes change (multiples of 4 and 8, 64, 256,
2048, 32768, 65536 and their neighbours). Everything is bit-exact against the CPU oracle, through
the C ABI, except Softmax forward (relative 1e-5).
"""
import numpy as np
import pytest

from checkers import MAX, MIN, SUM, Checker
from gpu_util import assert_bits_equal, f32, host_padded

pytestmark = pytest.mark.gpu

EDGE_WIDTHS = (4, 5, 7, 8, 9, 12, 13, 16, 27, 28, 31, 32, 55, 56, 63, 64, 65, 66, 100, 112, 127, 128,
               130, 255, 256, 257, 260)


@pytest.fixture(scope="module")
def G():
    import mshadow_amd
    g = mshadow_amd.load_cases()
    g.set_device(0)
    return g


@pytest.fixture(scope="module")
def stream(G):
    s = G.stream_create()
    yield s
    G.stream_destroy(s)


@pytest.fixture(scope="module")
def O():
    return Checker("orc")


def draw_size(rng, least):
    if rng.random() < 0.6:
        v = int(rng.choice(EDGE_WIDTHS))
    else:
        v = int(rng.integers(least, 140))
    return max(v, least)


@pytest.mark.parametrize("seed", range(120))
def test_pool_unpool_random_geometry(G, O, stream, seed):
    rng = np.random.default_rng(9000 + seed)
    ky, kx = (int(rng.integers(1, 5)),) * 2 if rng.random() < 0.7 else (int(rng.integers(1, 6)), int(rng.integers(1, 6)))
    sy, sx = (int(rng.integers(1, 4)),) * 2 if rng.random() < 0.8 else (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    h, w = draw_size(rng, ky), draw_size(rng, kx)
    if h * w > 20000:
        h = max(ky, 20000 // w)
    planes = int(rng.integers(1, max(2, min(600, 400000 // (h * w)))))
    pad = int(rng.choice((0, 0, 1, 3)))
    reducer = (MAX, MIN, SUM)[seed % 3]
    case = (planes, h, w, ky, kx, sy, sx, pad, reducer)
    # a coarse grid of values: equal maxima inside a window are common, zeros of both signs occur
    src = rng.integers(-6, 7, (planes, h, w)).astype(f32) / f32(4)
    src[rng.random(src.shape) < 0.02] = f32(-0.0)
    ph, pw = (h - ky) // sy + 1, (w - kx) // sx + 1
    if seed % 7 == 3 and ph > 1 and pw > 1:     # a pooled grid the caller names, smaller than the natural one
        ph, pw = ph - int(rng.integers(0, min(3, ph))), pw - int(rng.integers(0, min(3, pw)))
    want = np.empty((planes, ph, pw), f32)
    O.pool(want, host_padded(src, pad), ky, kx, sy, sx, reducer)
    dsrc = G.to_device(src, pad)
    dpool = G.buffer((planes, ph, pw), f32, pad)
    G.pool(dpool, dsrc, ky, kx, sy, sx, reducer, stream)
    assert_bits_equal(dpool.download(stream), want, f"pool {case}")
    grad = rng.standard_normal((planes, ph, pw)).astype(f32)
    wantu = np.empty((planes, h, w), f32)
    O.unpool(wantu, src, want, grad, ky, kx, sy, sx, reducer)
    dun = G.buffer((planes, h, w), f32, pad)
    G.unpool(dun, dsrc, dpool, G.to_device(grad, pad), ky, kx, sy, sx, reducer, stream)
    assert_bits_equal(dun.download(stream), wantu, f"unpool {case}")


@pytest.mark.parametrize("seed", range(100))
def test_im2col_col2im_random_geometry(G, O, stream, seed):
    rng = np.random.default_rng(7000 + seed)
    ky, kx = (int(rng.integers(1, 6)),) * 2 if rng.random() < 0.7 else (int(rng.integers(1, 6)), int(rng.integers(1, 6)))
    sy, sx = (1, 1) if rng.random() < 0.6 else (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    dy, dx = (1, 1) if rng.random() < 0.8 else (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    py, px = (int(rng.integers(0, 3)),) * 2 if rng.random() < 0.7 else (int(rng.integers(0, 4)), int(rng.integers(0, 4)))
    least_h = max(1, dy * (ky - 1) + 1 - 2 * py)
    least_w = max(1, dx * (kx - 1) + 1 - 2 * px)
    h, w = draw_size(rng, least_h), draw_size(rng, least_w)
    if h * w > 12000:
        h = max(least_h, 12000 // w)
    n, c = int(rng.integers(1, 4)), int(rng.integers(1, 5))
    dtype = "f16" if seed % 2 else "f32"
    cfg = (n, c, h, w, ky, kx, sy, sx, dy, dx, py, px, dtype)
    shape = Checker.col_shape(n, c, h, w, ky, kx, sy, sx, dy, dx, py, px)
    imgf = rng.uniform(-1, 1, (n, c, h, w)).astype(f32)
    colf = rng.standard_normal(shape).astype(f32)
    if dtype == "f16":
        img, colin, dt = O.float2half(imgf), O.float2half(colf), np.uint16
    else:
        img, colin, dt = imgf, colf, f32
    pad = int(rng.choice((0, 0, 3)))
    want = np.empty(shape, dt)
    O.im2col(want, img, ky, kx, sy, sx, dy, dx, py, px)
    dcol = G.buffer(shape, dt, pad)
    G.im2col(dcol, G.to_device(img, pad), ky, kx, sy, sx, dy, dx, py, px, stream)
    assert_bits_equal(dcol.download(stream), want, f"im2col {cfg}")
    wanti = np.empty((n, c, h, w), dt)
    O.col2im(wanti, colin, ky, kx, sy, sx, dy, dx, py, px)
    dimg = G.buffer((n, c, h, w), dt, pad)
    G.col2im(dimg, G.to_device(colin, pad), ky, kx, sy, sx, dy, dx, py, px, stream)
    assert_bits_equal(dimg.download(stream), wanti, f"col2im {cfg}")


ROW_LENGTHS = (1, 2, 3, 7, 31, 32, 33, 63, 64, 100, 255, 256, 257, 511, 513, 1000, 1023, 1024, 1025, 2047, 2048,
               2049, 4095, 4097, 8191, 8193, 16385, 32000, 32767, 32769, 50257, 65535, 65536, 65537, 70001)


@pytest.mark.parametrize("seed", range(60))
def test_softmax_random_shapes(G, O, stream, seed):
    """forward within 1e-5 of the CPU path (the tolerance of the task), gradient bit for bit, on row
    lengths drawn around the borders between the kernels, few rows or thousands, dense or pitched"""
    rng = np.random.default_rng(5000 + seed)
    cols = int(rng.choice(ROW_LENGTHS)) if rng.random() < 0.7 else int(rng.integers(1, 5000))
    rows = int(rng.integers(2048, 2600)) if (cols <= 2048 and seed % 3 == 0) else int(rng.integers(1, 12))
    pad = int(rng.choice((0, 0, 1, 2, 3)))
    shape = (rows, cols)
    x = (rng.standard_normal(shape) * rng.choice((0.5, 3.0, 12.0))).astype(f32)
    want = np.empty(shape, f32)
    O.softmax(want, x)
    dst = G.buffer(shape, f32, pad)
    G.softmax(dst, G.to_device(x, pad), stream)
    got = dst.download(stream)
    # relative 1e-5, the tolerance of the task; below the smallest normal number the difference is
    # measured against that number (a subnormal result has fewer than 24 bits to agree in)
    rel = np.abs(got.astype(np.float64) - want) / np.maximum(want, np.finfo(f32).tiny)
    assert rel.max() <= 1e-5, f"softmax {shape} pad {pad}: {rel.max():.3e}"
    label = rng.integers(0, cols, rows).astype(f32)
    wantg = np.empty(shape, f32)
    O.softmax_grad(wantg, want, label)
    dg = G.buffer(shape, f32, pad)
    G.softmax_grad(dg, G.to_device(want, pad), G.to_device(label), stream)
    assert_bits_equal(dg.download(stream), wantg, f"softmax_grad {shape} pad {pad}")


@pytest.mark.parametrize("seed", range(80))
def test_reductions_random_shapes(G, O, stream, seed):
    """sum_rows and sumall_except_dim<1> bit for bit (the kernels keep the CPU path's order of
    additions) on shapes drawn around the borders between their routes"""
    from checkers import MINUSTO, PLUSTO, SAVETO
    rng = np.random.default_rng(3000 + seed)
    reducer = (SUM, SUM, MAX, MIN)[seed % 4]
    saver, scale = ((SAVETO, 1.0), (PLUSTO, 0.75), (MINUSTO, 1.25))[seed % 3]
    pad = int(rng.choice((0, 0, 1, 3, 4)))
    if seed % 2 == 0:
        rows = int(rng.choice((1, 2, 63, 64, 65, 255, 256, 257, 1000, 4097)))
        cols = int(rng.choice((1, 3, 4, 15, 16, 17, 31, 32, 33, 64, 100, 255, 256, 1000, 4096, 4100)))
        if rows * cols > 1 << 21:
            rows = max(1, (1 << 21) // cols)
        m = rng.standard_normal((rows, cols)).astype(f32)
        start = rng.uniform(1, 3, cols).astype(f32)
        want = start.copy()
        O.reduce_keep_lowest(want, host_padded(m, pad), reducer, saver, scale)
        dst = G.to_device(start)
        G.reduce_keep_lowest(dst, G.to_device(m, pad), reducer, saver, scale, stream)
        assert_bits_equal(dst.download(stream), want, f"keep_lowest {(rows, cols)} pad {pad} seed {seed}")
    else:
        n = int(rng.choice((1, 2, 3, 15, 16, 17, 32, 33, 64, 70, 130)))
        c = int(rng.choice((1, 2, 3, 5, 16, 64, 200, 257)))
        h = int(rng.choice((1, 2, 7, 14, 16, 28, 33, 56)))
        w = int(rng.choice((1, 3, 4, 7, 8, 14, 16, 28, 36, 52, 56, 65)))
        while n * c * h * w > 1 << 21:
            if n > 2:
                n //= 2
            else:
                c = max(1, c // 2)
        x = rng.standard_normal((n, c, h, w)).astype(f32)
        start = rng.uniform(1, 3, c).astype(f32)
        want = start.copy()
        O.reduce_keep_highdim(want, host_padded(x, pad), reducer, saver, scale)
        dst = G.to_device(start)
        G.reduce_keep_highdim(dst, G.to_device(x, pad), reducer, saver, scale, stream)
        assert_bits_equal(dst.download(stream), want, f"keep_highdim {(n, c, h, w)} pad {pad} seed {seed}")
