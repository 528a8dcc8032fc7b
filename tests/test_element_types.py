"""Reductions and the softmax pair on half_t tensors: the oracle against the compiled reference
and against what 16-bit arithmetic fixes in closed form (CPU), and the HIP path against the
oracle (GPU).

half_t rounds after every operation (mshadow/half.h:45-66), so these functions are sensitive
to the order of the additions in a way the float ones are not: a sum of ones stops at 2048
(2048 + 1 is a tie that rounds to even), which no tree sum reproduces. Bars: bit-exact for the
reductions and the softmax gradient; Softmax forward within the task's relative 2e-3 for
half_t (observed: the only differences come from expf and are single roundings).
"""
import numpy as np
import pytest

from checkers import DIVTO, MAX, MIN, MINUSTO, MULTO, PLUSTO, SAVETO, SUM, Checker, have_ref

f32 = np.float32


def halves(orc, seed, shape, sigma=1.0):
    rng = np.random.default_rng(seed)
    return orc.float2half((rng.standard_normal(shape) * sigma).astype(f32))


# ------------------------------------------------------------------ CPU: oracle pinned
def test_half_sum_saturates_at_2048(orc):
    ones = orc.float2half(np.ones((5000, 3), f32))
    out = np.zeros(3, np.uint16)
    orc.reduce_keep_lowest(out, ones)
    assert orc.half2float(out).tolist() == [2048.0] * 3
    # order matters: 2048 first absorbs every later 1; the ones first reach 2050
    col = np.ones((3, 1), f32)
    col[0, 0] = 2048.0
    out1 = np.zeros(1, np.uint16)
    orc.reduce_keep_lowest(out1, orc.float2half(col))
    orc_rev = np.zeros(1, np.uint16)
    orc.reduce_keep_lowest(orc_rev, orc.float2half(col[::-1].copy()))
    assert orc.half2float(out1)[0] == 2048.0 and orc.half2float(orc_rev)[0] == 2050.0


def test_half_highdim_two_level_order(orc):
    # per kept index: inner sums over (y, x) per n, merged in n order. 3000 ones per n would
    # saturate a single running sum at 2048; two levels give 2 * 2048 = 4096
    src = orc.float2half(np.ones((2, 2, 30, 100), f32))
    out = np.zeros(2, np.uint16)
    orc.reduce_keep_highdim(out, src)
    assert orc.half2float(out).tolist() == [4096.0, 4096.0]
    orc.reduce_keep_highdim(out, src, reducer=MAX, scale=0.5)
    assert orc.half2float(out).tolist() == [0.5, 0.5]


def test_half_softmax_known_answers(orc):
    # n equal logits: every term is exactly 1; the half sum is n up to 2048 and stays there
    for n, denom in ((8, 8.0), (2048, 2048.0), (4096, 2048.0), (10000, 2048.0)):
        x = orc.float2half(np.full((2, n), 0.25, f32))
        p = np.empty_like(x)
        orc.softmax(p, x)
        assert np.all(orc.half2float(p) == f32(1.0 / denom)), n
    # gradient: half(p - 1) at static_cast<int>(label) (9.7 -> 9), a copy elsewhere and for
    # labels outside the row; multiples of 1/16 keep p - 1 exact
    p = orc.float2half((np.arange(40, dtype=f32) / 16).reshape(4, 10))
    lab = orc.float2half(np.array([3.0, 9.7, -1.0, 10.0], f32))
    g = np.empty_like(p)
    orc.softmax_grad(g, p, lab)
    d = orc.half2float(g) - orc.half2float(p)
    want = np.zeros((4, 10), f32)
    want[0, 3] = want[1, 9] = -1.0
    assert np.array_equal(d, want)
    # and a value where p - 1 has to round to 11 bits: 0.0769 - 1 = -0.9231 -> -0.92285
    q = orc.float2half(np.array([[0.0769]], f32))
    orc.softmax_grad(g[:1, :1], q, orc.float2half(np.zeros(1, f32)))
    assert g[0, 0] == orc.float2half(orc.half2float(q) - f32(1.0))[0, 0]


@pytest.mark.skipif(not have_ref(), reason="reference build absent")
@pytest.mark.parametrize("shape", [(1, 1), (7, 5), (300, 33), (5000, 4), (64, 1000)])
def test_half_oracle_equals_reference(orc, ref, shape):
    x = halves(orc, 7, shape, 3.0)
    a, b = np.empty_like(x), np.empty_like(x)
    orc.softmax(a, x)
    ref.softmax(b, x)
    assert np.array_equal(a, b)
    lab = orc.float2half(np.random.default_rng(8).integers(-1, shape[1] + 1, shape[0]).astype(f32))
    ga, gb = np.empty_like(x), np.empty_like(x)
    orc.softmax_grad(ga, a, lab)
    ref.softmax_grad(gb, a, lab)
    assert np.array_equal(ga, gb)
    for reducer in (SUM, MAX, MIN):
        for saver, scale in ((SAVETO, 1.0), (PLUSTO, 0.5), (MINUSTO, 3.0), (MULTO, 0.25), (DIVTO, 2.0)):
            oa = halves(orc, 9, (shape[1],))
            ob = oa.copy()
            orc.reduce_keep_lowest(oa, x, reducer, saver, scale)
            ref.reduce_keep_lowest(ob, x, reducer, saver, scale)
            assert np.array_equal(oa, ob), (reducer, saver)


@pytest.mark.skipif(not have_ref(), reason="reference build absent")
@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (3, 5, 7, 9), (20, 4, 30, 31)])
def test_half_highdim_oracle_equals_reference(orc, ref, shape):
    x = halves(orc, 11, shape)
    for reducer in (SUM, MAX, MIN):
        for saver, scale in ((SAVETO, 1.0), (PLUSTO, 0.5)):
            oa = halves(orc, 12, (shape[1],))
            ob = oa.copy()
            orc.reduce_keep_highdim(oa, x, reducer, saver, scale)
            ref.reduce_keep_highdim(ob, x, reducer, saver, scale)
            assert np.array_equal(oa, ob), (reducer, saver)


def test_half_map_and_pool_known_answers(orc):
    # a * b rounds before + c: 1.001 * 1.001 = 1.00195 in 16 bits, where the exact product
    # 1.0019541 + 2^-11 * 0.9 would round the sum differently
    a = orc.float2half(np.full((2, 3), 1.0009765625, f32))          # 1 + 2^-10
    c = orc.float2half(np.full((2, 3), 0.00048828125, f32))         # 2^-11
    out = np.empty_like(a)
    orc.map_muladd_f16(out, a, a, c)
    prod = orc.float2half(orc.half2float(a) * orc.half2float(a))     # 1 + 2^-9 (the 2^-20 is lost)
    assert np.all(orc.half2float(prod) == f32(1.001953125))
    assert np.array_equal(out, orc.float2half(orc.half2float(prod) + orc.half2float(c)))
    # pool<sum> of a 50 x 50 window of ones: the running 16-bit sum stops at 2048
    img = orc.float2half(np.ones((1, 50, 50), f32))
    o = np.empty((1, 1, 1), np.uint16)
    orc.pool(o, img, 50, 50, 1, 1, reducer=SUM)
    assert orc.half2float(o)[0, 0, 0] == 2048.0


@pytest.mark.skipif(not have_ref(), reason="reference build absent")
def test_half_map_and_pool_oracle_equals_reference(orc, ref):
    a, b, c = (halves(orc, 70 + i, (37, 53), 2.0) for i in range(3))
    for saver in (SAVETO, PLUSTO, MINUSTO, MULTO, DIVTO):
        oa = halves(orc, 73, (37, 53))
        ob = oa.copy()
        orc.map_muladd_f16(oa, a, b, c, saver)
        ref.map_muladd_f16(ob, a, b, c, saver)
        assert np.array_equal(oa, ob), saver
    img = halves(orc, 74, (3, 4, 23, 29))
    for reducer in (SUM, MAX, MIN):
        for (ky, kx, sy, sx) in ((3, 3, 2, 2), (2, 5, 1, 3)):
            shape = (3, 4, (23 - ky) // sy + 1, (29 - kx) // sx + 1)
            pa, pb = np.empty(shape, np.uint16), np.empty(shape, np.uint16)
            orc.pool(pa, img, ky, kx, sy, sx, reducer)
            ref.pool(pb, img, ky, kx, sy, sx, reducer)
            assert np.array_equal(pa, pb), (reducer, ky, kx)


# ------------------------------------------------------------------ GPU parity
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


def _bits(orc, scale):
    return int(orc.float2half(np.array([scale], f32))[0])


@pytest.mark.gpu
@pytest.mark.parametrize("shape,pad", [((1, 1), 0), ((5000, 3), 0), ((300, 33), 5), ((4096, 130), 0),
                                       ((17, 1000), 2),
                                       # long columns: several stages of the large workgroup, a ragged last
                                       # stage, fewer columns than a strip, even and odd pitches
                                       ((2048, 2), 0), ((5000, 64), 2), ((6001, 36), 0), ((3000, 100), 3),
                                       ((5000, 4), 0)])
def test_gpu_half_reduce_keep_lowest(G, orc, stream, shape, pad):
    x = halves(orc, 21, shape)
    if shape in ((5000, 3), (5000, 4)):
        x = orc.float2half(np.ones(shape, f32))       # saturates at 2048 only in row order
    src = G.to_device(x, pad)
    for variant in (0, 1):
        for reducer in (SUM, MAX, MIN):
            for saver, scale in ((SAVETO, 1.0), (PLUSTO, 0.5), (DIVTO, 2.0)):
                init = halves(orc, 22, (shape[1],))
                want = init.copy()
                orc.reduce_keep_lowest(want, x, reducer, saver, scale)
                dst = G.to_device(init)
                G.case_reduce_keep_lowest(dst, src, reducer, saver, _bits(orc, scale), variant, stream)
                got = dst.download(stream)
                assert np.array_equal(got, want), (variant, reducer, saver)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,pad", [((1, 1, 1, 1), 0), ((3, 5, 7, 9), 3), ((2, 2, 30, 100), 0),
                                       ((20, 6, 28, 28), 0),
                                       # enough work per kept index for the LDS-ring kernel: 64, 16, 4
                                       # and 1 segments side by side, ragged last stages, an even pad
                                       # (taken) and an odd one (falls back to the generic kernel)
                                       ((64, 5, 56, 56), 0), ((70, 3, 33, 30), 2), ((6, 3, 150, 100), 0),
                                       ((3, 2, 301, 128), 6), ((1, 2, 700, 100), 0), ((20, 3, 60, 62), 3),
                                       ((33, 2, 40, 51), 1),
                                       # pitched rows of whole 16-byte packs: the inner chains in
                                       # groups of 16 segments, as for the dense shapes above
                                       ((36, 5, 40, 48), 8)])
def test_gpu_half_reduce_keep_highdim(G, orc, stream, shape, pad):
    x = halves(orc, 31, shape)
    if shape == (2, 2, 30, 100):
        x = orc.float2half(np.ones(shape, f32))       # 4096 only with the two-level order
    src = G.to_device(x, pad)
    for variant in (0, 1):
        for reducer in (SUM, MAX, MIN):
            for saver, scale in ((SAVETO, 1.0), (MINUSTO, 0.5)):
                init = halves(orc, 32, (shape[1],))
                want = init.copy()
                orc.reduce_keep_highdim(want, x, reducer, saver, scale)
                dst = G.to_device(init)
                G.case_reduce_keep_highdim(dst, src, reducer, saver, _bits(orc, scale), variant, stream)
                assert np.array_equal(dst.download(stream), want), (variant, reducer, saver)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,pad", [((1, 1), 0), ((7, 5), 0), ((9, 513), 3), ((64, 1000), 0),
                                       ((5, 4096), 0), ((3, 32000), 0), ((130, 77), 1)])
def test_gpu_half_softmax(G, orc, stream, shape, pad):
    x = halves(orc, 41, shape, 3.0)
    if shape == (5, 4096):
        x = orc.float2half(np.full(shape, 0.25, f32))  # 1/2048 each: the sum saturates
    want = np.empty_like(x)
    orc.softmax(want, x)
    src = G.to_device(x, pad)
    dst = G.buffer(shape, np.uint16, pad)
    G.case_softmax(dst, src, stream)
    got = dst.download(stream)
    w, g = orc.half2float(want).astype(np.float64), orc.half2float(got).astype(np.float64)
    differ = int(np.count_nonzero(got != want))
    # relative 2e-3 for values above the smallest normal half (one subnormal ulp below it)
    tol = np.maximum(2e-3 * np.abs(w), 2.0 ** -24)
    assert np.all(np.abs(g - w) <= tol), np.max(np.abs(g - w) / np.maximum(np.abs(w), 2.0 ** -14))
    if shape == (5, 4096):
        assert differ == 0 and np.all(g == 1.0 / 2048)
    print(f"half softmax {shape}: {differ} of {got.size} outputs differ from the CPU path")
    # in place
    G.case_softmax(src, src, stream)
    assert np.array_equal(src.download(stream), got)
    # gradient: bit-exact, labels inside, on the edge and outside the row
    lab = orc.float2half(np.random.default_rng(42).integers(-1, shape[1] + 1, shape[0]).astype(f32))
    gw = np.empty_like(got)
    orc.softmax_grad(gw, got, lab)
    gd = G.buffer(shape, np.uint16, pad)
    G.case_softmax_grad(gd, src, G.to_device(lab), stream)
    assert np.array_equal(gd.download(stream), gw)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 1), (33, 1000), (4, 20000)])
def test_gpu_double_softmax(G, stream, shape):
    """Softmax on double tensors: the same left-to-right sum in double, against numpy's
    float64 evaluation of the same steps (parity unpinned at the ulp level: the device and
    the host exponential are different libraries)"""
    rng = np.random.default_rng(51)
    x = rng.standard_normal(shape) * 3.0
    t = np.exp(x - x.max(axis=1, keepdims=True))
    s = np.zeros(shape[0])
    for j in range(shape[1]):
        s = s + t[:, j]
    want = t / s[:, None]
    dst = G.buffer(shape, np.float64)
    G.case_softmax(dst, G.to_device(x), stream)
    got = dst.download(stream)
    assert np.all(np.abs(got - want) <= 1e-13 * want + 1e-300)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,pad", [((1, 1), 0), ((37, 53), 3), ((256, 1024), 0), ((33, 4096), 0)])
def test_gpu_half_map(G, orc, stream, shape, pad):
    """dst <saver>= a * b + c on half_t tensors through the generic expression kernels, bit-exact"""
    a, b, c = (halves(orc, 80 + i, shape, 2.0) for i in range(3))
    da, db, dc = (G.to_device(t, pad) for t in (a, b, c))
    for saver in (SAVETO, PLUSTO, MINUSTO, MULTO, DIVTO):
        init = halves(orc, 83, shape)
        want = init.copy()
        orc.map_muladd_f16(want, a, b, c, saver)
        dst = G.to_device(init, pad)
        G.case_map_muladd_f16(dst, da, db, dc, saver, stream)
        assert np.array_equal(dst.download(stream), want), saver


@pytest.mark.gpu
@pytest.mark.parametrize("window", [(3, 3, 2, 2), (2, 5, 1, 3), (50, 50, 1, 1)])
def test_gpu_half_pool(G, orc, stream, window):
    ky, kx, sy, sx = window
    img = halves(orc, 90, (3, 4, 56, 61))
    if window == (50, 50, 1, 1):
        img = orc.float2half(np.ones((3, 4, 56, 61), f32))   # sums stop at 2048 in window order
    shape = (3, 4, (56 - ky) // sy + 1, (61 - kx) // sx + 1)
    src = G.to_device(img)
    for reducer in (SUM, MAX, MIN):
        want = np.empty(shape, np.uint16)
        orc.pool(want, img, ky, kx, sy, sx, reducer)
        dst = G.buffer(shape, np.uint16)
        G.case_pool(dst, src, ky, kx, sy, sx, reducer, 0, stream)
        assert np.array_equal(dst.download(stream), want), reducer


@pytest.mark.gpu
@pytest.mark.parametrize("shape,pad,kind", [
    ((3, 32000), 0, "equal"),        # every term counts until the sum stops: too many for the list
    ((4, 31999), 1, "normal"),       # ragged rows, odd pitch
    ((6, 4100), 4, "normal"),        # just above the shortest row this kernel takes
    ((5, 8192), 8, "normal"),        # pitched rows of whole packs
    ((2, 32768), 0, "normal"),       # the longest row it takes
    ((2, 32769), 0, "normal"),       # one more: several rows per workgroup again
    ((3, 20000), 0, "ascending"),    # the largest term comes last: the bound stays low
    ((3, 20000), 0, "descending"),   # ... comes first
    ((3, 24000), 0, "spike"),        # one class far above the others
    ((2, 16000), 0, "tiny")])        # terms that are all subnormal or zero but one
def test_gpu_half_softmax_long_rows(G, orc, stream, shape, pad, kind):
    """rows of 4096 .. 32768 half_t are kept on chip and their sum is built from the terms that
    can still change it (mshadow/hip/kernels/half_prune.h): bit-identical to the CPU path's
    term-by-term sum whatever the row looks like"""
    rng = np.random.default_rng(hash(kind) % 1000 + shape[1])
    x = rng.standard_normal(shape, dtype=f32) * f32(3)
    if kind == "equal":
        x[:] = f32(0.25)
    elif kind == "ascending":
        x = np.sort(x, axis=1)
    elif kind == "descending":
        x = -np.sort(-x, axis=1)
    elif kind == "spike":
        x[np.arange(shape[0]), rng.integers(0, shape[1], shape[0])] += f32(30)
    elif kind == "tiny":
        x = x - f32(14)
        x[:, 5000] = f32(3)
    x = orc.float2half(x)
    want = np.empty_like(x)
    orc.softmax(want, x)
    src = G.to_device(x, pad)
    dst = G.buffer(shape, np.uint16, pad)
    G.case_softmax(dst, src, stream)
    got = dst.download(stream)
    differ = int(np.count_nonzero(got != want))
    w, g = orc.half2float(want).astype(np.float64), orc.half2float(got).astype(np.float64)
    tol = np.maximum(2e-3 * np.abs(w), 2.0 ** -24)
    assert np.all(np.abs(g - w) <= tol), (kind, differ)
    if kind == "equal":
        assert differ == 0 and np.all(g == 1.0 / 2048)
    print(f"half softmax {shape} {kind}: {differ} of {got.size} outputs differ from the CPU path")
    # the sum itself, free of the exponential: the library's terms, summed by the CPU path's loop
    G.case_softmax(src, src, stream)   # in place
    assert np.array_equal(src.download(stream), got)


@pytest.mark.gpu
def test_gpu_half_softmax_full_size(G, orc, stream):
    """8192 x 32000 half_t logits N(0, 3): forward within relative 2e-3 of the CPU path (the
    differences counted and printed; none observed), the gradient bit for bit, and the
    size-independent property that the gradient differs from the probabilities at the label
    of each row and nowhere else"""
    rows, cols = 8192, 32000
    x = orc.float2half(np.random.default_rng(7).standard_normal((rows, cols), dtype=f32) * f32(3))
    want = np.empty_like(x)
    orc.softmax(want, x)
    src = G.to_device(x)
    dst = G.buffer(x.shape, np.uint16)
    G.case_softmax(dst, src, stream)
    got = dst.download(stream)
    differ = got != want
    print(f"half softmax {x.shape}: {int(differ.sum())} of {got.size} outputs differ from the CPU path")
    if differ.any():
        w = orc.half2float(want[differ]).astype(np.float64)
        g = orc.half2float(got[differ]).astype(np.float64)
        assert np.all(np.abs(g - w) <= np.maximum(2e-3 * np.abs(w), 2.0 ** -24))
    lab = orc.float2half(np.random.default_rng(8).integers(0, 2049, rows).astype(f32))
    gd = G.buffer(x.shape, np.uint16)
    G.case_softmax_grad(gd, dst, G.to_device(lab), stream)
    grad = gd.download(stream)
    gw = np.empty_like(got)
    orc.softmax_grad(gw, got, lab)
    assert np.array_equal(grad, gw)
    changed = np.argwhere(grad != got)
    assert np.array_equal(changed[:, 0], np.arange(rows))
    assert np.array_equal(changed[:, 1], orc.half2float(lab).astype(np.int64))


@pytest.mark.gpu
def test_gpu_half_reductions_full_size(G, orc, stream):
    """the two reductions on half_t at the BASELINE shapes, bit for bit against the CPU path (the
    compiled reference where it is present): sumall_except_dim<1> over (64,256,56,56) through the
    LDS-ring kernel, sum_rows over 16384 x 4096 through the generic one"""
    chk = Checker("ref") if have_ref() else orc
    x4 = halves(orc, 71, (64, 256, 56, 56))
    src4 = G.to_device(x4)
    for reducer in (SUM, MAX):
        want = np.zeros(256, np.uint16)
        chk.reduce_keep_highdim(want, x4, reducer, SAVETO, 1.0)
        dst = G.buffer((256,), np.uint16)
        G.case_reduce_keep_highdim(dst, src4, reducer, SAVETO, _bits(orc, 1.0), 0, stream)
        assert np.array_equal(dst.download(stream), want), reducer
    m = halves(orc, 72, (16384, 4096))
    want = np.zeros(4096, np.uint16)
    chk.reduce_keep_lowest(want, m, SUM, SAVETO, 1.0)
    dst = G.buffer((4096,), np.uint16)
    G.case_reduce_keep_lowest(dst, G.to_device(m), SUM, SAVETO, _bits(orc, 1.0), 0, stream)
    assert np.array_equal(dst.download(stream), want)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 1), (5000, 7), (300, 130), (3, 5, 7, 9), (20, 6, 28, 28)])
def test_gpu_double_reductions(G, stream, shape):
    """sum_rows / sumall_except_dim<1> (and max, min) on double tensors through the generic
    reduction kernels, bit for bit against the CPU path's order restated with numpy's
    sequential float64 accumulate (mshadow/tensor_cpu-inl.h:203-268)"""
    x = np.random.default_rng(61).standard_normal(shape)
    src = G.to_device(x)
    if len(shape) == 2:
        want = {SUM: np.add.accumulate(x, axis=0)[-1], MAX: x.max(axis=0), MIN: x.min(axis=0)}
        keep = shape[1]
    else:
        n, c, h, w = shape
        inner = np.add.accumulate(x.transpose(1, 0, 2, 3).reshape(c, n, h * w), axis=2)[:, :, -1]
        want = {SUM: np.add.accumulate(inner, axis=1)[:, -1], MAX: x.max(axis=(0, 2, 3)),
                MIN: x.min(axis=(0, 2, 3))}
        keep = c
    for reducer in (SUM, MAX, MIN):
        dst = G.buffer((keep,), np.float64)
        G.case_reduce_f64(dst, src, reducer, 0.5, stream)
        got = dst.download(stream)
        assert np.array_equal(got, want[reducer] * 0.5), reducer


# mshadow::TypeFlag codes (mshadow/base.h:306-316) and what numpy calls the type
TYPE_FLAGS = [(0, np.float32), (1, np.float64), (2, np.float16), (3, np.uint8), (4, np.int32),
              (5, np.int8), (6, np.int64)]


@pytest.mark.gpu
@pytest.mark.parametrize("flag,dtype", TYPE_FLAGS)
@pytest.mark.parametrize("shape", [(1, 3), (37, 53), (64, 1024)])
def test_gpu_map_every_element_type(G, stream, flag, dtype, shape):
    """dst = a * b + c and dst = pad(crop(a, ...), 1) for every element type of
    MSHADOW_TYPE_SWITCH through the generic expression kernels, bit for bit against numpy
    (integer types wrap modulo their width on the store, as the C++ conversion does; float16
    rounds the product before the sum, as half_t does)"""
    rng = np.random.default_rng(100 + flag)
    if np.issubdtype(dtype, np.floating):
        a, b, c = (rng.standard_normal(shape).astype(dtype) for _ in range(3))
        want = (a * b).astype(dtype) + c
    else:
        a, b, c = (rng.integers(-50 if np.issubdtype(dtype, np.signedinteger) else 0, 50, shape)
                   .astype(dtype) for _ in range(3))
        wide = a.astype(np.int64) * b.astype(np.int64) + c.astype(np.int64)
        want = wide.astype(dtype)      # modulo 2^bits, like the conversion on the store
    da, db, dc = (G.to_device(t) for t in (a, b, c))
    dst = G.buffer(shape, dtype)
    G.case_map_any(0, flag, dst, da, db, dc, stream)
    got = dst.download(stream)
    assert np.array_equal(got.view(np.uint8), np.ascontiguousarray(want).view(np.uint8))
    if shape[0] > 2:
        G.case_map_any(1, flag, dst, da, db, dc, stream)
        want = np.zeros(shape, dtype)
        want[1:-1, 1:-1] = a[1:-1, 1:-1]
        assert np.array_equal(dst.download(stream), want)
