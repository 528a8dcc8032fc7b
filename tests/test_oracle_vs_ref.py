"""Bit-for-bit agreement of the C restatement with the reference's own headers.

oracle/_ref/libmshadow_ref.so is dmlc/mshadow compiled from /root/reference (see
oracle/Makefile); it exists only where that tree is present, otherwise these tests skip.
Seeded random inputs at sizes that run in seconds, padded strides included, every saver
and reducer. Equality is on the raw bits.
"""
import numpy as np
import pytest

from checkers import (DIVTO, MAX, MIN, MINUSTO, MULTO, PLUSTO, SAVETO, SUM, Checker, padded)

f32 = np.float32


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32 if a.dtype == f32 else np.uint16)


def same(a, b):
    return np.array_equal(bits(a), bits(b))


def rnd(rng, shape, pad=0, kind="uniform"):
    out = padded(shape, f32, pad, fill=np.nan)
    out[...] = rng.uniform(-1, 1, shape) if kind == "uniform" else rng.standard_normal(shape)
    return out


def test_half_conversions_all_floats_sampled(orc, ref):
    rng = np.random.default_rng(10)
    x = rng.integers(0, 2**32, size=4_000_000, dtype=np.uint64).astype(np.uint32).view(f32)
    x = x[~np.isnan(x)]
    assert np.array_equal(orc.float2half(x), ref.float2half(x))
    x = (rng.standard_normal(1_000_000) * 1e-5).astype(f32)  # subnormal-heavy
    assert np.array_equal(orc.float2half(x), ref.float2half(x))
    h = np.arange(65536, dtype=np.uint16)
    a, b = orc.half2float(h), ref.half2float(h)
    ok = ~np.isnan(a)
    assert same(a[ok], b[ok]) and np.array_equal(np.isnan(a), np.isnan(b))


@pytest.mark.parametrize("saver", [SAVETO, PLUSTO, MINUSTO, MULTO, DIVTO])
@pytest.mark.parametrize("pad", [0, 3])
def test_map_fused(orc, ref, saver, pad):
    rng = np.random.default_rng(11 + saver)
    shape = (257, 515)
    a, b, c, d = (rnd(rng, shape, pad) for _ in range(4))
    start = rng.uniform(1, 2, shape).astype(f32)
    o1, o2 = padded(shape, f32, pad), padded(shape, f32, pad)
    o1[...] = start
    o2[...] = start
    orc.map_fused(o1, a, b, c, d, saver)
    ref.map_fused(o2, a, b, c, d, saver)
    assert same(o1, o2)


def test_map_fused_wide_range_sigmoid(orc, ref):
    rng = np.random.default_rng(12)
    shape = (64, 1024)
    a, b, d = (rnd(rng, shape) for _ in range(3))
    c = (rng.standard_normal(shape) * 40).astype(f32)  # exercises the clamp of the functor
    o1, o2 = np.empty(shape, f32), np.empty(shape, f32)
    orc.map_fused(o1, a, b, c, d)
    ref.map_fused(o2, a, b, c, d)
    assert same(o1, o2)


def test_map_scalar_and_axpb(orc, ref):
    rng = np.random.default_rng(13)
    for saver in (SAVETO, PLUSTO, MULTO, DIVTO):
        o1 = rnd(rng, (33, 65), 1)
        o2 = o1.base.copy()[:, :65]
        orc.map_scalar(o1, 1.7, saver)
        ref.map_scalar(o2, 1.7, saver)
        assert same(o1, o2)
        a = rnd(rng, (33, 65))
        orc.map_axpb(o1, a, 10.0, 3.0, 2.0, saver)
        ref.map_axpb(o2, a, 10.0, 3.0, 2.0, saver)
        assert same(o1, o2)


@pytest.mark.parametrize("reducer", [SUM, MAX, MIN])
@pytest.mark.parametrize("saver", [SAVETO, PLUSTO, MINUSTO, MULTO, DIVTO])
def test_reductions(orc, ref, reducer, saver):
    rng = np.random.default_rng(20 + reducer * 5 + saver)
    m = rnd(rng, (2049, 131), 5, kind="normal")
    start = rng.uniform(1, 2, 131).astype(f32)
    o1, o2 = start.copy(), start.copy()
    orc.reduce_keep_lowest(o1, m, reducer, saver, 0.75)
    ref.reduce_keep_lowest(o2, m, reducer, saver, 0.75)
    assert same(o1, o2)
    x = rnd(rng, (9, 17, 23, 29), 3, kind="normal")
    start = rng.uniform(1, 2, 17).astype(f32)
    o1, o2 = start.copy(), start.copy()
    orc.reduce_keep_highdim(o1, x, reducer, saver, 1.25)
    ref.reduce_keep_highdim(o2, x, reducer, saver, 1.25)
    assert same(o1, o2)


def test_reduction_config_like_shapes(orc, ref):
    rng = np.random.default_rng(30)
    x = rng.standard_normal((8, 32, 56, 56)).astype(f32)
    o1, o2 = np.empty(32, f32), np.empty(32, f32)
    orc.reduce_keep_highdim(o1, x)
    ref.reduce_keep_highdim(o2, x)
    assert same(o1, o2)
    m = rng.standard_normal((16384, 256)).astype(f32)
    o1, o2 = np.empty(256, f32), np.empty(256, f32)
    orc.reduce_keep_lowest(o1, m)
    ref.reduce_keep_lowest(o2, m)
    assert same(o1, o2)


@pytest.mark.parametrize("pad", [0, 7])
def test_softmax_and_grad(orc, ref, pad):
    rng = np.random.default_rng(40 + pad)
    src = padded((65, 32000), f32, pad)
    src[...] = rng.standard_normal((65, 32000)) * 3
    o1, o2 = padded(src.shape, f32, pad), padded(src.shape, f32, pad)
    orc.softmax(o1, src)
    ref.softmax(o2, src)
    assert same(o1, o2)
    label = rng.integers(-3, 32003, 65).astype(f32)
    g1, g2 = np.empty(src.shape, f32), np.empty(src.shape, f32)
    orc.softmax_grad(g1, o1, label)
    ref.softmax_grad(g2, o2, label)
    assert same(g1, g2)
    # in place
    i1, i2 = src.copy(), src.copy()
    orc.softmax(i1, i1)
    ref.softmax(i2, i2)
    assert same(i1, i2) and same(i1, o1)


@pytest.mark.parametrize("cfg", [(3, 3, 2, 2), (2, 2, 2, 2), (3, 2, 1, 3), (5, 5, 3, 2), (1, 1, 1, 1)])
@pytest.mark.parametrize("reducer", [MAX, MIN, SUM])
def test_pool_unpool(orc, ref, cfg, reducer):
    ky, kx, sy, sx = cfg
    rng = np.random.default_rng(50 + ky * 7 + kx + reducer)
    planes, h, w = 6, 37, 41
    # few distinct values -> many duplicated maxima, which equality routing must honour
    src = padded((planes, h, w), f32, 2)
    src[...] = rng.integers(-4, 5, (planes, h, w)).astype(f32) / 4
    ph, pw = (h - ky) // sy + 1, (w - kx) // sx + 1
    p1, p2 = padded((planes, ph, pw), f32, 1), padded((planes, ph, pw), f32, 1)
    orc.pool(p1, src, ky, kx, sy, sx, reducer)
    ref.pool(p2, src, ky, kx, sy, sx, reducer)
    assert same(p1, p2)
    grad = rnd(rng, (planes, ph, pw), 0, kind="normal")
    u1, u2 = np.empty((planes, h, w), f32), np.empty((planes, h, w), f32)
    orc.unpool(u1, src, p1, grad, ky, kx, sy, sx, reducer)
    ref.unpool(u2, src, p2, grad, ky, kx, sy, sx, reducer)
    assert same(u1, u2)


@pytest.mark.parametrize("cfg", [(3, 3, 2, 2), (2, 2, 1, 1), (3, 3, 1, 1)])
@pytest.mark.parametrize("reducer", [MAX, MIN, SUM])
def test_pool_special_values(orc, ref, cfg, reducer):
    """NaN, infinities, zeros of both signs and the largest finite values as window members: std::max /
    std::min pass over a NaN and keep the first of two equal zeros"""
    ky, kx, sy, sx = cfg
    rng = np.random.default_rng(90 + ky + sy + reducer)
    src = (rng.integers(-3, 4, (5, 21, 23)).astype(f32) / 2)
    flat = src.reshape(-1)
    specials = np.array([np.nan, np.inf, -np.inf, -0.0, 0.0, 3.4028235e38, -3.4028235e38, 1e-45, -1e-45], f32)
    where = rng.random(flat.size) < 0.3
    flat[where] = specials[rng.integers(0, specials.size, int(where.sum()))]
    flat[:60] = np.nan  # windows of NaN only
    ph, pw = (21 - ky) // sy + 1, (23 - kx) // sx + 1
    p1, p2 = np.empty((5, ph, pw), f32), np.empty((5, ph, pw), f32)
    orc.pool(p1, src, ky, kx, sy, sx, reducer)
    ref.pool(p2, src, ky, kx, sy, sx, reducer)
    assert same(p1, p2)


CONV = [(3, 3, 1, 1, 1, 1, 1, 1), (3, 3, 2, 2, 1, 1, 0, 0), (5, 3, 2, 1, 1, 1, 2, 1),
        (3, 3, 1, 1, 2, 2, 2, 2), (2, 3, 1, 2, 2, 2, 1, 0), (3, 3, 2, 2, 2, 1, 2, 2),
        (1, 1, 1, 1, 1, 1, 0, 0), (7, 7, 3, 3, 1, 1, 3, 3)]


@pytest.mark.parametrize("cfg", CONV)
@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_im2col_col2im(orc, ref, cfg, dtype):
    ky, kx, sy, sx, dy, dx, py, px = cfg
    rng = np.random.default_rng(60 + sum(cfg))
    n, c, h, w = 3, 5, 19, 23
    shape = Checker.col_shape(n, c, h, w, ky, kx, sy, sx, dy, dx, py, px)
    imgf = rng.uniform(-1, 1, (n, c, h, w)).astype(f32)
    colf = rng.standard_normal(shape).astype(f32)
    if dtype == "f16":
        img, colin = orc.float2half(imgf), orc.float2half(colf)
        dt = np.uint16
    else:
        img, colin, dt = imgf, colf, f32
    c1, c2 = np.empty(shape, dt), np.empty(shape, dt)
    orc.im2col(c1, img, ky, kx, sy, sx, dy, dx, py, px)
    ref.im2col(c2, img, ky, kx, sy, sx, dy, dx, py, px)
    assert same(c1, c2)
    i1, i2 = np.empty((n, c, h, w), dt), np.empty((n, c, h, w), dt)
    orc.col2im(i1, colin, ky, kx, sy, sx, dy, dx, py, px)
    ref.col2im(i2, colin, ky, kx, sy, sx, dy, dx, py, px)
    assert same(i1, i2)


def test_col2im_half_config_like(orc, ref):
    # the convolution shape of the benchmark in small: (2,16,56,56) k3 s1 pad1 in half, N(0,1) columns
    rng = np.random.default_rng(70)
    n, c, h, w = 2, 16, 56, 56
    shape = Checker.col_shape(n, c, h, w, 3, 3, 1, 1, 1, 1, 1, 1)
    col = orc.float2half(rng.standard_normal(shape).astype(f32))
    i1, i2 = np.empty((n, c, h, w), np.uint16), np.empty((n, c, h, w), np.uint16)
    orc.col2im(i1, col, 3, 3, 1, 1, 1, 1, 1, 1)
    ref.col2im(i2, col, 3, 3, 1, 1, 1, 1, 1, 1)
    assert same(i1, i2)
    # float accumulation rounded once would differ on a large share of pixels
    acc = np.empty((n, c, h, w), f32)
    orc.col2im(acc, orc.half2float(col), 3, 3, 1, 1, 1, 1, 1, 1)
    assert np.mean(orc.float2half(acc) != i1) > 0.2
