"""Known-answer and closed-form checks that pin the C restatement (oracle/oracle.c).

Sources of the fixed values are the reference's own test programs and documentation
(cited per test); the rest are mathematical identities chosen so that a dropped term,
a transposed index or a wrong rounding point fails at least one of them.
"""
import math
import os

import numpy as np
import pytest

from checkers import (DIVTO, MAX, MIN, MINUSTO, MULTO, PLUSTO, SAVETO, SUM, Checker, padded)

GOLD = os.path.join(os.path.dirname(__file__), "golden")
f32 = np.float32


# ---------------------------------------------------------------- half
def test_half_roundtrip_exhaustive(orc):
    h = np.arange(65536, dtype=np.uint16)
    f = orc.half2float(h)
    back = orc.float2half(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], h[~nan])
    assert np.all((back[nan] & 0x7c00) == 0x7c00) and np.all((back[nan] & 0x3ff) != 0)
    # agrees with IEEE binary16 as numpy implements it
    assert np.array_equal(f[~nan].view(np.uint32), h[~nan].view(np.float16).astype(f32).view(np.uint32))


def test_half_rne_structured(orc):
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    # add ties, denormal boundaries, overflow edge, extremes
    special = np.array([0x33000000, 0x33000001, 0x33800000, 0x387fffff, 0x38800000, 0x477fe000,
                        0x477fefff, 0x477ff000, 0x47800000, 0x7f800000, 0x3f801000, 0x3f803000,
                        0x3f802fff, 0x3f803001, 0x00000001, 0x80000000, 0x38000000, 0x387fe000,
                        0x33c00000], dtype=np.uint32)
    bits = np.concatenate([bits, special, special | 0x80000000])
    x = bits.view(f32)
    ok = ~np.isnan(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = orc.float2half(x)
    assert np.array_equal(got[ok], want[ok])
    # MSHADOW_HALF_MIN / MAX bit patterns (mshadow/half.h:350-351)
    assert orc.half2float(np.array([0xFBFF, 0x7BFF], dtype=np.uint16)).tolist() == [-65504.0, 65504.0]


# ---------------------------------------------------------------- map
def test_map_basic_guide_values(orc):
    # guide/basic.cpp:21-27: mat = 0; mat[0][1] = 1; mat[1][0] = 2; mat += (mat + 10) / 10 + 2
    mat = np.zeros((2, 5), dtype=f32)
    orc.map_scalar(mat, 0.0)
    mat[0, 1], mat[1, 0] = 1.0, 2.0
    src = mat.copy()
    orc.map_axpb(mat, src, 10.0, 10.0, 2.0, saver=PLUSTO)
    want = src + ((src + f32(10)) / f32(10) + f32(2))
    assert np.array_equal(mat, want)
    assert mat[0, 0] == f32(3.0) and abs(mat[0, 1] - 4.1) < 1e-6 and abs(mat[1, 0] - 5.2) < 1e-6


def _sigmoid_bruteforce(c):
    """pmath_sigmoid restated with numpy float32 scalar ops (independent of the C build)."""
    x = -c.astype(f32)
    x = np.minimum(np.maximum(x, f32(-87.0)), f32(88.0))
    kf = x * f32(1.44269502162933349609375)
    k = (kf + np.where(kf < 0, f32(-0.5), f32(0.5))).astype(np.int32)
    fk = k.astype(f32)
    r = x - fk * f32(0.693145751953125)
    r = r - fk * f32(1.428606765330187045e-06)
    p = np.full_like(r, f32(1.9841270113829523e-04))
    for coef in (1.3888889225199819e-03, 8.3333337679505348e-03, 4.1666667908430099e-02,
                 1.6666667163372040e-01, 0.5, 1.0, 1.0):
        p = p * r + f32(coef)
    s = ((k + 127).astype(np.uint32) << np.uint32(23)).view(f32)
    e = p * s
    return f32(1.0) / (f32(1.0) + e)


def test_map_fused_bruteforce_and_accuracy(orc):
    rng = np.random.default_rng(1)
    shape = (37, 129)
    a, b, c, d = (rng.uniform(-1, 1, shape).astype(f32) for _ in range(4))
    dst = np.empty(shape, f32)
    orc.map_fused(dst, a, b, c, d)
    want = ((a * b) + (f32(0.5) * _sigmoid_bruteforce(c))) - d
    assert np.array_equal(dst.view(np.uint32), want.view(np.uint32))
    # the functor is a faithful sigmoid (accuracy, not parity)
    exact = a.astype(np.float64) * b + 0.5 / (1 + np.exp(-c.astype(np.float64))) - d
    assert np.max(np.abs(dst - exact)) < 1e-6
    # wrong parenthesisation would differ somewhere on this many elements
    alt = (a * b) + ((f32(0.5) * _sigmoid_bruteforce(c)) - d)
    assert not np.array_equal(alt, want)


def test_map_savers_and_stride(orc):
    rng = np.random.default_rng(2)
    shape = (5, 7)
    a, b, c, d = (rng.uniform(-1, 1, shape).astype(f32) for _ in range(4))
    base = np.empty(shape, f32)
    orc.map_fused(base, a, b, c, d)
    for saver, op in ((PLUSTO, np.add), (MINUSTO, np.subtract), (MULTO, np.multiply),
                      (DIVTO, np.divide)):
        dst = padded(shape, f32, 3, fill=7.0)
        start = rng.uniform(1, 2, shape).astype(f32)
        dst[...] = start
        orc.map_fused(dst, a, b, c, d, saver=saver)
        assert np.array_equal(dst, op(start, base))
        assert np.all(dst.base[:, 7:] == 7.0)  # padding untouched


# ---------------------------------------------------------------- reductions
def _tc():
    # test/test.cu:9-18
    i, j, k = np.meshgrid(np.arange(3), np.arange(2), np.arange(4), indexing="ij")
    return (f32(0.1) * i.astype(f32) + f32(0.2) * j.astype(f32) + f32(0.1) * k.astype(f32)).astype(f32)


def test_reduce_reference_test_values(orc):
    tc = _tc()
    out = np.empty(4, f32)
    orc.reduce_keep_lowest(out, tc[0])  # test/test.cu:35 sum_rows(tc[0])
    assert np.allclose(out, [0.2, 0.4, 0.6, 0.8], atol=1e-4)  # EPS of test/test.h:7
    out3 = np.empty(3, f32)
    # test/test.cu:47 sumall_except_dim<0>(tc): shape viewed as (1, 3, 2, 4)
    orc.reduce_keep_highdim(out3, tc.reshape(1, 3, 2, 4))
    assert np.allclose(out3, [2.0, 2.8, 3.6], atol=1e-4)


def test_reduce_doc_examples(orc):
    # doc/README.md:162-168: dst(=1) += sumall_except_dim<1>(src*2), src = ones(2,3,2) -> 9
    src = np.full((2, 3, 2, 1), 2.0, f32).reshape(2, 3, 2, 1)
    dst = np.ones(3, f32)
    orc.reduce_keep_highdim(dst, src, saver=PLUSTO)
    assert dst.tolist() == [9.0, 9.0, 9.0]
    # doc/README.md:179-185: dst(=1) += sum_rows(ones(3,2) + 1) -> 7
    dst = np.ones(2, f32)
    orc.reduce_keep_lowest(dst, np.full((3, 2), 2.0, f32), saver=PLUSTO)
    assert dst.tolist() == [7.0, 7.0]


def test_reduce_order_is_sequential(orc):
    # values chosen so that any other association changes the float result
    col = np.array([1e8, 1.0, -1e8, 1.0, 3.0, 1e-3], dtype=f32)
    want = f32(0)
    seq = col[0]
    for v in col[1:]:
        seq = f32(seq + v)
    src = np.stack([col, col[::-1]], axis=1).copy()
    out = np.empty(2, f32)
    orc.reduce_keep_lowest(out, src)
    seq2 = src[0, 1]
    for v in src[1:, 1]:
        seq2 = f32(seq2 + v)
    assert out[0] == seq and out[1] == seq2 and seq != seq2
    # high-dim: inner (y,x) sums start from 0 per n, then merged over n
    x4 = np.stack([col, col[::-1]]).reshape(2, 1, 2, 3)
    t = []
    for n in range(2):
        s = f32(0)
        for v in x4[n, 0].ravel():
            s = f32(s + v)
        t.append(s)
    want = f32(f32(f32(0) + t[0]) + t[1])
    o = np.empty(1, f32)
    orc.reduce_keep_highdim(o, x4)
    assert o[0] == want


def test_reduce_counts_scale_and_reducers(orc):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 6, 7, 9)).astype(f32)
    ones = np.ones_like(x)
    o = np.empty(6, f32)
    orc.reduce_keep_highdim(o, ones)
    assert np.all(o == 5 * 7 * 9)
    orc.reduce_keep_highdim(o, x, reducer=MAX)
    assert np.array_equal(o, x.max(axis=(0, 2, 3)))
    orc.reduce_keep_highdim(o, x, reducer=MIN, scale=2.0)
    assert np.array_equal(o, x.min(axis=(0, 2, 3)) * f32(2))
    m = x.reshape(-1, 9)
    o9 = np.empty(9, f32)
    orc.reduce_keep_lowest(o9, m, reducer=MAX)
    assert np.array_equal(o9, m.max(axis=0))
    orc.reduce_keep_lowest(o9, m, scale=0.5)
    assert np.allclose(o9, m.astype(np.float64).sum(axis=0) * 0.5, rtol=0, atol=1e-4)


# ---------------------------------------------------------------- softmax
def test_softmax_uniform_and_invariants(orc):
    for n in (4, 7, 1000):
        src = np.full((3, n), 0.37, f32)
        dst = np.empty_like(src)
        orc.softmax(dst, src)
        assert np.all(dst == f32(1.0) / f32(n))
    rng = np.random.default_rng(4)
    src = (rng.standard_normal((6, 513)) * 3).astype(f32)
    dst = np.empty_like(src)
    orc.softmax(dst, src)
    x64 = src.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    want = e / e.sum(axis=1, keepdims=True)
    assert np.max(np.abs(dst - want) / want) < 5e-6
    assert np.allclose(dst.sum(axis=1), 1.0, atol=1e-5)
    # monotone in the logits
    order = np.argsort(src, axis=1)
    assert np.all(np.diff(np.take_along_axis(dst, order, axis=1), axis=1) >= 0)
    # in place equals out of place (tensor_cpu-inl.h:278-283 reads before writing)
    inplace = src.copy()
    orc.softmax(inplace, inplace)
    assert np.array_equal(inplace, dst)
    # power-of-two shift of the logits: x - max is unchanged when exact
    dst2 = np.empty_like(src)
    ints = rng.integers(-8, 8, size=src.shape).astype(f32)
    orc.softmax(dst, ints)
    orc.softmax(dst2, ints + f32(16))
    assert np.array_equal(dst, dst2)


def test_softmax_sum_is_left_to_right(orc):
    # one row whose float sum depends on the order of addition
    rng = np.random.default_rng(5)
    src = (rng.standard_normal((1, 20000)) * 3).astype(f32)
    dst = np.empty_like(src)
    orc.softmax(dst, src)
    p = np.exp((src[0] - src[0].max()).astype(f32))  # numpy float32 exp: close, not identical
    # reconstruct the sum the oracle used from its own outputs: p_i / sum, largest p is 1
    s = f32(1.0) / dst[0, np.argmax(src[0])]
    seq = f32(0)
    for v in p:
        seq = f32(seq + v)
    pair = p.astype(f32).sum(dtype=f32)  # numpy pairwise
    assert abs(float(s) - float(seq)) / float(seq) < 2e-6
    # the sequential sum is measurably different from an accurate one on this size
    assert abs(float(seq) - float(p.astype(np.float64).sum())) / float(seq) > 2e-6 or pair == seq


def test_softmax_grad(orc):
    rng = np.random.default_rng(6)
    src = rng.uniform(0, 1, (9, 33)).astype(f32)
    label = rng.integers(0, 33, 9).astype(f32)
    label[3] = 40.0   # outside: plain copy
    label[4] = -2.0
    label[5] = 7.9    # truncates to 7
    dst = np.empty_like(src)
    orc.softmax_grad(dst, src, label)
    diff = dst - src
    for y in range(9):
        k = int(label[y])
        for x in range(33):
            assert diff[y, x] == (f32(-1.0) if x == k else 0.0)
        if not 0 <= k < 33:
            assert np.array_equal(dst[y], src[y])


# ---------------------------------------------------------------- pool / unpool
def test_pool_reference_test_values(orc):
    # test/pool.cu:29-48 and test/pairtest.cu:29-53: 6x6 0.1i+0.1j, 2x2 stride 2 max
    i, j = np.meshgrid(np.arange(6), np.arange(6), indexing="ij")
    src = (i.astype(f32) * f32(0.1) + j.astype(f32) * f32(0.1)).reshape(1, 6, 6)
    out = np.empty((1, 3, 3), f32)
    orc.pool(out, src, 2, 2, 2, 2)
    assert np.array_equal(out[0], src[0, 1::2, 1::2])
    # 7x7 ramp 7i+j, 3x3 stride 2: out[a][b] = 7(2a+2) + (2b+2)
    src = (7 * np.arange(7)[:, None] + np.arange(7)[None, :]).astype(f32).reshape(1, 7, 7)
    out = np.empty((1, 3, 3), f32)
    orc.pool(out, src, 3, 3, 2, 2)
    a, b = np.meshgrid(np.arange(3), np.arange(3), indexing="ij")
    assert np.array_equal(out[0], (7 * (2 * a + 2) + (2 * b + 2)).astype(f32))
    assert out[0, 0, 0] == 16


def test_pool_sum_of_upsampled(orc):
    # guide/basic.cpp:127-134: pool<sum> with k = stride = 3 of a 3x nearest upsampling = 9 * small
    small = np.arange(6, dtype=f32).reshape(1, 2, 3)
    up = np.repeat(np.repeat(small, 3, axis=1), 3, axis=2).copy()
    out = np.empty_like(small)
    orc.pool(out, up, 3, 3, 3, 3, reducer=SUM)
    assert np.array_equal(out, 9 * small)


def test_pool_bruteforce_clipped_and_strided(orc):
    rng = np.random.default_rng(7)
    src = padded((4, 9, 11), f32, 2)
    src[...] = rng.uniform(-1, 1, (4, 9, 11))
    for (ky, kx, sy, sx, ph, pw) in ((3, 3, 2, 2, 4, 5), (2, 3, 1, 2, 8, 5), (3, 2, 3, 1, 4, 10)):
        out = np.empty((4, ph, pw), f32)
        orc.pool(out, src, ky, kx, sy, sx)
        for p in range(4):
            for a in range(ph):
                for b in range(pw):
                    win = src[p, a * sy:min(a * sy + ky, 9), b * sx:min(b * sx + kx, 11)]
                    # an explicit pshape may ask for windows past the edge: they keep the
                    # reducer's initial value (spatial_pool.h:137, base.h:794-797)
                    assert out[p, a, b] == (win.max() if win.size else -np.finfo(f32).max)
        orc.pool(out, src, ky, kx, sy, sx, reducer=MIN)
        assert out[1, 1, 1] == src[1, sy:sy + ky, sx:sx + kx].min()


def test_unpool_reference_test_values(orc):
    # test/pairtest.cu:60-77: grad 0.1 lands exactly on the window maxima (2a+1, 2b+1)
    i, j = np.meshgrid(np.arange(6), np.arange(6), indexing="ij")
    src = (i.astype(f32) * f32(0.1) + j.astype(f32) * f32(0.1)).reshape(1, 6, 6)
    pooled = np.empty((1, 3, 3), f32)
    orc.pool(pooled, src, 2, 2, 2, 2)
    grad = np.full((1, 3, 3), 0.1, f32)
    out = np.empty_like(src)
    orc.unpool(out, src, pooled, grad, 2, 2, 2, 2)
    want = np.zeros_like(src)
    want[0, 1::2, 1::2] = f32(0.1)
    assert np.array_equal(out, want)


def test_unpool_properties(orc):
    rng = np.random.default_rng(8)
    src = rng.permutation(4 * 11 * 13).astype(f32).reshape(4, 11, 13)  # unique values
    ky = kx = 3
    sy = sx = 2
    ph, pw = (11 - ky) // sy + 1, (13 - kx) // sx + 1
    pooled = np.empty((4, ph, pw), f32)
    orc.pool(pooled, src, ky, kx, sy, sx)
    grad = rng.integers(-4, 5, size=pooled.shape).astype(f32)
    out = np.empty_like(src)
    orc.unpool(out, src, pooled, grad, ky, kx, sy, sx)
    # unique maxima: total gradient is conserved, and it sits on arg-max positions
    assert out.sum() == grad.sum()
    want = np.zeros_like(src)
    for p in range(4):
        for a in range(ph):
            for b in range(pw):
                win = src[p, a * sy:a * sy + ky, b * sx:b * sx + kx]
                yy, xx = np.unravel_index(np.argmax(win), win.shape)
                want[p, a * sy + yy, b * sx + xx] += grad[p, a, b]
    assert np.array_equal(out, want)
    # duplicated maximum: equality routing gives the gradient to both (spatial_unpool.h:117-121)
    s = np.zeros((1, 3, 3), f32)
    s[0, 0, 0] = s[0, 2, 2] = 5.0
    pl = np.empty((1, 1, 1), f32)
    orc.pool(pl, s, 3, 3, 1, 1)
    o = np.empty_like(s)
    orc.unpool(o, s, pl, np.full((1, 1, 1), 2.0, f32), 3, 3, 1, 1)
    assert o[0, 0, 0] == 2.0 and o[0, 2, 2] == 2.0 and o.sum() == 4.0
    # rows / cols no window covers stay zero (112 -> 55 with k3 s2 leaves the last one out)
    src = rng.uniform(-1, 1, (2, 12, 12)).astype(f32)
    pooled = np.empty((2, 5, 5), f32)
    orc.pool(pooled, src, 3, 3, 2, 2)
    out = np.empty_like(src)
    orc.unpool(out, src, pooled, np.ones_like(pooled), 3, 3, 2, 2)
    assert np.all(out[:, 11, :] == 0) and np.all(out[:, :, 11] == 0)


# ---------------------------------------------------------------- im2col / col2im
def test_im2col_reference_test_values(orc):
    # test/unpack.cu:29-59: 6x6 0.1i+0.2j, k3 s2: col[ky*3+kx][oy*2+ox] = src[2oy+ky][2ox+kx]
    i, j = np.meshgrid(np.arange(6), np.arange(6), indexing="ij")
    img = (i.astype(f32) * f32(0.1) + j.astype(f32) * f32(0.2)).reshape(1, 1, 6, 6)
    col = np.empty((9, 4), f32)
    orc.im2col(col, img, 3, 3, 2, 2)
    for ky in range(3):
        for kx in range(3):
            for oy in range(2):
                for ox in range(2):
                    assert col[ky * 3 + kx, oy * 2 + ox] == img[0, 0, 2 * oy + ky, 2 * ox + kx]


def _im2col_brute(img, ky, kx, sy, sx, dy, dx, py, px):
    n, c, h, w = img.shape
    p = np.zeros((n, c, h + 2 * py, w + 2 * px), img.dtype)
    p[:, :, py:py + h, px:px + w] = img
    oh = (h + 2 * py - (dy * (ky - 1) + 1)) // sy + 1
    ow = (w + 2 * px - (dx * (kx - 1) + 1)) // sx + 1
    col = np.zeros((c * ky * kx, n * oh * ow), img.dtype)
    for ci in range(c):
        for a in range(ky):
            for b in range(kx):
                for ni in range(n):
                    for oy in range(oh):
                        for ox in range(ow):
                            col[(ci * ky + a) * kx + b, (ni * oh + oy) * ow + ox] = \
                                p[ni, ci, oy * sy + a * dy, ox * sx + b * dx]
    return col


@pytest.mark.parametrize("cfg", [(3, 3, 1, 1, 1, 1, 1, 1), (3, 2, 2, 1, 1, 1, 0, 2),
                                 (2, 3, 1, 2, 2, 2, 1, 0), (3, 3, 2, 2, 2, 1, 2, 2)])
def test_im2col_index_valued(orc, cfg):
    ky, kx, sy, sx, dy, dx, py, px = cfg
    n, c, h, w = 2, 3, 7, 8
    img = (np.arange(n * c * h * w, dtype=np.uint16) + 1).reshape(n, c, h, w)  # self-describing
    shape = Checker.col_shape(n, c, h, w, ky, kx, sy, sx, dy, dx, py, px)
    col = np.empty(shape, np.uint16)
    orc.im2col(col, img, ky, kx, sy, sx, dy, dx, py, px)
    assert np.array_equal(col, _im2col_brute(img, ky, kx, sy, sx, dy, dx, py, px))
    imgf = img.astype(f32)
    colf = np.empty(shape, f32)
    orc.im2col(colf, imgf, ky, kx, sy, sx, dy, dx, py, px)
    assert np.array_equal(colf, col.astype(f32))


def test_col2im_coverage_counts(orc):
    # all-ones columns, k3 s1 pad1: each pixel counts the patches covering it: 4 / 6 / 9
    n, c, h, w = 1, 2, 5, 6
    shape = Checker.col_shape(n, c, h, w, 3, 3, 1, 1, 1, 1, 1, 1)
    one = orc.float2half(np.ones(shape, f32))
    img = np.empty((n, c, h, w), np.uint16)
    orc.col2im(img, one, 3, 3, 1, 1, 1, 1, 1, 1)
    got = orc.half2float(img)
    want = np.full((h, w), 9.0, f32)
    want[0, :] = want[-1, :] = want[:, 0] = want[:, -1] = 6.0
    want[0, 0] = want[0, -1] = want[-1, 0] = want[-1, -1] = 4.0
    assert np.array_equal(got[0, 0], want) and np.array_equal(got[0, 1], want)


# pack_col2patch steps py/px by the dilation (pack_col2patch.h:133-134), which visits
# exactly the covering patches when the stride is 1 or the dilation is 1; those are the
# configurations where it is the mathematical adjoint of unpack_patch2col.
@pytest.mark.parametrize("cfg", [(3, 3, 1, 1, 1, 1, 1, 1), (3, 2, 2, 1, 1, 1, 0, 2),
                                 (2, 3, 1, 1, 2, 2, 1, 0), (3, 3, 2, 2, 1, 1, 2, 2),
                                 (3, 3, 1, 1, 2, 1, 2, 2)])
def test_col2im_is_adjoint_of_im2col(orc, cfg):
    ky, kx, sy, sx, dy, dx, py, px = cfg
    n, c, h, w = 2, 2, 7, 9
    rng = np.random.default_rng(9)
    x = rng.integers(-3, 4, (n, c, h, w)).astype(f32)
    shape = Checker.col_shape(n, c, h, w, ky, kx, sy, sx, dy, dx, py, px)
    cmat = rng.integers(-3, 4, shape).astype(f32)
    ux = np.empty(shape, f32)
    orc.im2col(ux, x, ky, kx, sy, sx, dy, dx, py, px)
    pc = np.empty((n, c, h, w), f32)
    orc.col2im(pc, cmat, ky, kx, sy, sx, dy, dx, py, px)
    assert float((ux.astype(np.float64) * cmat).sum()) == float((x.astype(np.float64) * pc).sum())
    # small integers are exact in half too: the half path must agree with the float path
    pch = np.empty((n, c, h, w), np.uint16)
    orc.col2im(pch, orc.float2half(cmat), ky, kx, sy, sx, dy, dx, py, px)
    assert np.array_equal(orc.half2float(pch), pc)


def test_col2im_half_rounds_every_step(orc):
    # k3 s1 pad1, centre pixel of a 3x3 image: 9 terms in (py, px) order. Values are
    # chosen so that rounding to half after each add differs from rounding once.
    n, c, h, w = 1, 1, 3, 3
    shape = Checker.col_shape(n, c, h, w, 3, 3, 1, 1, 1, 1, 1, 1)
    terms = np.array([2048.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0], f32)
    col = np.zeros(shape, f32)
    # centre (y=1,x=1) in padded coords (2,2): patch (py,px) contributes row (2-py)*3 + (2-px)
    for idx, (py, px) in enumerate((a, b) for a in range(3) for b in range(3)):
        col[(2 - py) * 3 + (2 - px), py * 3 + px] = terms[idx]
    img = np.empty((n, c, h, w), np.uint16)
    orc.col2im(img, orc.float2half(col), 3, 3, 1, 1, 1, 1, 1, 1)
    centre = orc.half2float(img)[0, 0, 1, 1]
    assert centre == 2048.0      # each +1 is half an ulp at 2048 and ties to even
    assert f32(terms.sum()) == 2056.0  # a single final rounding would have given 2056
