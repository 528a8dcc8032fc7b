"""The softmax gradient family, the 3-D softmax and the row scatter / gather functions on
element types other than float (double, half_t) and on index vectors other than int32 / float
(int64, half_t): mshadow/tensor_cpu-inl.h:286-528, templated over DType and IndexType there
and in mshadow/tensor_gpu-inl.h:157-240.

CPU: the C restatement (`orc_*_any`) is pinned three ways - against numpy evaluating the same
expressions with the same roundings (float16 / float64 arithmetic is IEEE in numpy, so this is
a second, independent statement of where each type rounds), against the functions already
pinned for float and for the 2-D half softmax, and against the reference's own templates
compiled from its headers. GPU: the HIP path against the restatement. Bars: bit-exact for the
gradients and the row functions in every type; the 3-D Softmax forward within relative 2e-3
(half_t) / 1e-13 (double), the only differences coming from the exponential.
"""
import numpy as np
import pytest

from checkers import GRAD_IGNORE, GRAD_SMOOTH, Checker, have_ref

f16, f32, f64 = np.float16, np.float32, np.float64
DTYPES = [f32, f64, f16]
INDEX_TYPES = [np.int32, np.int64, f32, f16]


def probs(seed, shape, dtype):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(shape) * 2.0
    e = np.exp(x - x.max(axis=1 if len(shape) > 1 else 0, keepdims=True))
    return (e / e.sum(axis=1, keepdims=True)).astype(dtype)


def labels(seed, shape, classes, dtype):
    # inside the row, on its edges and outside it; .7 fractions exercise the truncation
    rng = np.random.default_rng(seed)
    lab = rng.integers(-1, classes + 1, shape).astype(f64) + 0.7 * (rng.random(shape) < 0.3)
    return lab.astype(dtype)


def numpy_grad(p, lab, flags, ignore, alpha, axis):
    """the host expressions in numpy, one rounding per operation of the element type"""
    dt = p.dtype
    classes = p.shape[axis]
    k = lab.astype(f32 if dt != f64 else f64).astype(np.int64)   # static_cast<int>(label)
    ignore_k = int(dt.type(f32(ignore)))
    smooth = f32(alpha) / f32(classes - 1)
    idx = np.arange(classes).reshape([-1 if a == axis else 1 for a in range(p.ndim)])
    at = idx == np.expand_dims(k, axis)
    wide = f64 if dt == f64 else f32

    def op(a, b, fn):     # DType OP float -> DType: compute widened, round to the element type
        return fn(a.astype(wide), wide(b)).astype(dt)
    hit = op(p, f32(1.0), np.subtract)
    other = p
    if flags & GRAD_SMOOTH:
        hit = op(hit, f32(alpha), np.add)
        other = op(p, smooth, np.subtract)
    out = np.where(at, hit, other)
    if flags & GRAD_IGNORE:
        out = np.where(np.expand_dims(k == ignore_k, axis), dt.type(0), out)
    return out.astype(dt)


# ------------------------------------------------------------------ CPU: oracle pinned
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("flags", [0, 1, 2, 3])
@pytest.mark.parametrize("shape", [(1, 2), (37, 53), (5, 3, 7), (4, 21, 33)])
def test_grad_family_matches_numpy_roundings(orc, dtype, flags, shape):
    p = probs(3, shape, dtype)
    lshape = (shape[0],) if len(shape) == 2 else (shape[0], shape[2])
    lab = labels(4, lshape, shape[1], dtype)
    ignore, alpha = float(lab.flat[0]), 0.1
    got = orc.grad_family_any(np.empty_like(p), p, lab, flags, ignore, alpha)
    want = numpy_grad(p, lab, flags, ignore, alpha, axis=1)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_grad_family_float_equals_pinned_float_functions(orc):
    p, lab = probs(5, (40, 17), f32), labels(6, (40,), 17, f32)
    p3, lab3 = probs(7, (6, 9, 11), f32), labels(8, (6, 11), 9, f32)
    for flags in range(4):
        a = orc.grad_family_any(np.empty_like(p), p, lab, flags, 3.0, 0.2)
        b = orc.softmax_grad_ex(np.empty_like(p), p, lab, flags, 3.0, 0.2)
        assert np.array_equal(a, b)
        a3 = orc.grad_family_any(np.empty_like(p3), p3, lab3, flags, 2.0, 0.3)
        b3 = orc.softmax3d_grad(np.empty_like(p3), p3, lab3, flags, 2.0, 0.3)
        assert np.array_equal(a3, b3)


def test_half_grad_rounds_after_every_operation(orc):
    # p = 2^-12: p - 1 is a tie between 1 - 2^-11 and 1 and rounds to -1 (even); adding
    # alpha = 2^-11 then gives -(1 - 2^-11). One rounding of p - 1 + alpha = -(1 - 2^-11 - 2^-12)
    # would instead be a tie that goes to -(1 - 2^-10)... the two differ, which pins the order.
    p = np.array([[2.0 ** -12, 0.5]], f16)
    lab = np.array([0.0], f16)
    got = orc.grad_family_any(np.empty_like(p), p, lab, GRAD_SMOOTH, 0.0, 2.0 ** -11)
    assert float(got[0, 0]) == -(1.0 - 2.0 ** -11)
    once = f16(f32(p[0, 0]) - f32(1.0) + f32(2.0 ** -11))
    assert float(once) != float(got[0, 0])
    # the other column: 0.5 - alpha / (2 - 1), one rounding
    assert float(got[0, 1]) == float(f16(f32(0.5) - f32(2.0 ** -11)))


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 7), (2, 40, 33), (4, 300, 2)])
def test_softmax3d_half_is_the_2d_softmax_of_the_transposed_tensor(orc, shape):
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(shape) * 3).astype(f16)
    got = orc.softmax3d_any(np.empty_like(x), x)
    d0, d1, d2 = shape
    rows = np.ascontiguousarray(x.transpose(0, 2, 1).reshape(d0 * d2, d1)).view(np.uint16)
    want = np.empty_like(rows)
    orc.softmax(want, rows)   # the 2-D half_t Softmax, pinned elsewhere
    want = want.view(f16).reshape(d0, d2, d1).transpose(0, 2, 1)
    assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(want).view(np.uint16))


def test_softmax3d_half_sum_saturates(orc):
    # 4096 equal logits along the middle axis: every term is 1, the half sum stops at 2048
    x = np.full((2, 4096, 3), 0.25, f16)
    got = orc.softmax3d_any(np.empty_like(x), x)
    assert np.all(got.astype(f64) == 1.0 / 2048)


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 7), (2, 40, 33)])
def test_softmax3d_double_against_numpy(orc, shape):
    rng = np.random.default_rng(12)
    x = rng.standard_normal(shape) * 3
    got = orc.softmax3d_any(np.empty_like(x), x)
    t = np.exp(x - x.max(axis=1, keepdims=True))
    s = np.zeros((shape[0], shape[2]))
    for j in range(shape[1]):
        s = s + t[:, j, :]
    want = t / s[:, None, :]
    assert np.all(np.abs(got - want) <= 4e-16 * want)
    xf = x.astype(f32)
    assert np.array_equal(orc.softmax3d_any(np.empty_like(xf), xf), orc.softmax3d(np.empty_like(xf), xf))


def numpy_rows_by_index(op, dst, sorted_rows, index, src):
    out = dst.copy()
    wide = f64 if dst.dtype == f64 else f32
    to_int = lambda v: int(f32(v)) if v.dtype == f16 else int(v)   # noqa: E731
    for y in range(index.shape[0]):
        if op == 0:
            j, frm = min(max(to_int(index[y]), 0), dst.shape[0] - 1), y
        elif op == 1:
            j, frm = to_int(sorted_rows[y]), to_int(index[y])
        else:
            j, frm = to_int(index[y]), y
        if op == 2:
            out[j] = src[frm]
        else:
            out[j] = (out[j].astype(wide) + src[frm].astype(wide)).astype(dst.dtype)
    return out


def row_case(seed, dtype, itype, op, k_rows=23, n_index=400, cols=37):
    rng = np.random.default_rng(seed)
    dst = rng.standard_normal((k_rows, cols)).astype(dtype)
    src = rng.standard_normal((n_index, cols)).astype(dtype)
    lo, hi = (-3, k_rows + 3) if op == 0 else (0, k_rows)      # AddTakeGrad clamps
    index = rng.integers(lo, hi, n_index).astype(itype)
    sorted_rows = None
    if op == 1:
        sorted_rows = np.sort(rng.integers(0, k_rows, n_index)).astype(itype)
        index = rng.integers(0, n_index, n_index).astype(itype)
    return dst, sorted_rows, index, src


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("itype", INDEX_TYPES)
@pytest.mark.parametrize("op", [0, 1, 2])
def test_rows_by_index_matches_numpy_roundings(orc, dtype, itype, op):
    dst, srt, index, src = row_case(21 + op, dtype, itype, op)
    want = numpy_rows_by_index(op, dst, srt, index, src)
    got = orc.rows_by_index_any(op, dst.copy(), srt, index, src)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_half_row_sum_depends_on_the_order(orc):
    # 2048 + 1 + 1 in half_t is 2048 (each +1 is a tie to even); 1 + 1 + 2048 is 2050
    src = np.array([[2048.0], [1.0], [1.0]], f16)
    index = np.zeros(3, np.int32)
    a = orc.rows_by_index_any(0, np.zeros((1, 1), f16), None, index, src)
    b = orc.rows_by_index_any(0, np.zeros((1, 1), f16), None, index, src[::-1].copy())
    assert float(a[0, 0]) == 2048.0 and float(b[0, 0]) == 2050.0


@pytest.mark.skipif(not have_ref(), reason="reference build absent")
@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_equals_reference_templates(orc, ref, dtype):
    for shape in [(1, 2), (37, 53), (300, 7), (5, 3, 7), (4, 21, 33)]:
        p = probs(31, shape, dtype)
        lshape = (shape[0],) if len(shape) == 2 else (shape[0], shape[2])
        lab = labels(32, lshape, shape[1], dtype)
        for flags in range(4):
            a = orc.grad_family_any(np.empty_like(p), p, lab, flags, float(lab.flat[-1]), 0.15)
            b = ref.grad_family_any(np.empty_like(p), p, lab, flags, float(lab.flat[-1]), 0.15)
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (shape, flags)
    for shape in [(1, 1, 1), (3, 5, 7), (2, 40, 33), (2, 3000, 2)]:
        x = (np.random.default_rng(33).standard_normal(shape) * 3).astype(dtype)
        a = orc.softmax3d_any(np.empty_like(x), x)
        b = ref.softmax3d_any(np.empty_like(x), x)
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), shape
    for itype in INDEX_TYPES:
        for op in range(3):
            dst, srt, index, src = row_case(34 + op, dtype, itype, op)
            a = orc.rows_by_index_any(op, dst.copy(), srt, index, src)
            b = ref.rows_by_index_any(op, dst.copy(), srt, index, src)
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (itype, op)


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


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,pad", [((1, 2), 0), ((37, 53), 3), ((130, 2048), 0), ((3, 33000), 0),
                                       ((5, 3, 7), 1), ((4, 21, 33), 0), ((2, 5, 4096), 0)])
def test_gpu_grad_family(G, orc, stream, dtype, shape, pad):
    p = probs(41, shape, dtype)
    lshape = (shape[0],) if len(shape) == 2 else (shape[0], shape[2])
    lab = labels(42, lshape, shape[1], dtype)
    src, dl = G.to_device(p, pad), G.to_device(lab, pad if len(lshape) == 2 else 0)
    for flags in range(4):
        ignore = float(lab.flat[0])
        want = orc.grad_family_any(np.empty_like(p), p, lab, flags, ignore, 0.1)
        dst = G.buffer(shape, dtype, pad)
        G.case_grad_family_any(dst, src, dl, flags, ignore, 0.1, stream)
        got = dst.download(stream)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), flags
    # in place
    want = orc.grad_family_any(np.empty_like(p), p, lab, 3, float(lab.flat[0]), 0.1)
    G.case_grad_family_any(src, src, dl, 3, float(lab.flat[0]), 0.1, stream)
    assert np.array_equal(src.download(stream).view(np.uint8), want.view(np.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [f16, f64])
@pytest.mark.parametrize("shape,pad", [((1, 1, 1), 0), ((3, 5, 7), 2), ((2, 40, 33), 0), ((2, 4096, 3), 0),
                                       ((16, 21, 1000), 0)])
def test_gpu_softmax3d(G, orc, stream, dtype, shape, pad):
    x = (np.random.default_rng(43).standard_normal(shape) * 3).astype(dtype)
    if shape == (2, 4096, 3):
        x[...] = 0.25        # half_t: the sum saturates at 2048
    want = orc.softmax3d_any(np.empty_like(x), x)
    src = G.to_device(x, pad)
    dst = G.buffer(shape, dtype, pad)
    G.case_softmax3d_any(dst, src, stream)
    got = dst.download(stream)
    w, g = want.astype(f64), got.astype(f64)
    if dtype == f16:
        tol = np.maximum(2e-3 * np.abs(w), 2.0 ** -24)
        if shape == (2, 4096, 3):
            assert np.array_equal(got, want) and np.all(g == 1.0 / 2048)
    else:
        tol = 1e-13 * np.abs(w) + 1e-300
    assert np.all(np.abs(g - w) <= tol)
    print(f"{np.dtype(dtype).name} softmax3d {shape}: {int(np.count_nonzero(got != want))} of {got.size} differ")
    G.case_softmax3d_any(src, src, stream)   # in place
    assert np.array_equal(src.download(stream).view(np.uint8), got.view(np.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("itype", INDEX_TYPES)
@pytest.mark.parametrize("op", [0, 1, 2])
def test_gpu_rows_by_index(G, orc, stream, dtype, itype, op):
    for k_rows, n_index, cols, pad in ((23, 400, 37, 3), (1, 5, 1, 0), (700, 3000, 130, 0)):
        if itype == f16 and max(k_rows, n_index) > 2048:
            k_rows, n_index = 700, 2000      # integers a half_t holds exactly
        dst, srt, index, src = row_case(51 + op, dtype, itype, op, k_rows, n_index, cols)
        want = orc.rows_by_index_any(op, dst.copy(), srt, index, src)
        d = G.to_device(dst, pad)
        G.case_rows_by_index_any(op, d, G.to_device(srt) if srt is not None else None,
                                 G.to_device(index), G.to_device(src, pad), stream)
        got = d.download(stream)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (k_rows, n_index, cols)


# ------------------------------------------------------------------ SortByKey, any types
def stable_order(keys, ascend):
    """positions in the order std::stable_sort gives under `<` (ascending) or `>` (descending):
    by key, equal keys (-0.0 and +0.0 are equal) in their original order"""
    _, rank = np.unique(keys, return_inverse=True)
    return np.lexsort((np.arange(keys.shape[0]), rank if ascend else -rank))


def sort_case(seed, ktype, vtype, n):
    rng = np.random.default_rng(seed)
    if np.issubdtype(ktype, np.floating):
        keys = np.round(rng.standard_normal(n) * 4, 1).astype(ktype)    # many repeated keys
        keys[rng.integers(0, n, max(n // 50, 1))] = -0.0
        keys[rng.integers(0, n, max(n // 50, 1))] = 0.0
        if n > 10:
            keys[:4] = [np.inf, -np.inf, np.finfo(ktype).max, np.finfo(ktype).tiny]
    else:
        info = np.iinfo(ktype)
        keys = rng.integers(max(info.min, -300), min(info.max, 300), n, endpoint=True).astype(ktype)
        if n > 10:
            keys[:2] = [info.min, info.max]
    wrap = {1: 251, 2: 2039}.get(np.dtype(vtype).itemsize, n + 1)   # values the narrow types hold exactly
    values = (np.arange(n) % wrap).astype(vtype)
    return keys, values


SORT_TYPES = [(f64, np.int32), (np.int64, f32), (f64, f64), (np.int64, np.uint8), (np.uint8, np.int64),
              (np.int8, f32), (f32, f64), (np.int32, f16), (f32, np.int32)]


@pytest.mark.skipif(not have_ref(), reason="reference build absent")
@pytest.mark.parametrize("ktype,vtype", SORT_TYPES)
@pytest.mark.parametrize("ascend", [True, False])
def test_stable_order_model_is_what_the_reference_sorts(ref, ktype, vtype, ascend):
    keys, values = sort_case(61, ktype, vtype, 3000)
    order = stable_order(keys, ascend)
    k, v = ref.sort_by_key_any(keys.copy(), values.copy(), ascend)
    assert np.array_equal(k.view(np.uint8), keys[order].view(np.uint8))
    assert np.array_equal(v.view(np.uint8), values[order].view(np.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("ktype,vtype", SORT_TYPES)
@pytest.mark.parametrize("ascend", [True, False])
@pytest.mark.parametrize("n", [1, 2, 777, 100000])
def test_gpu_sort_by_key_any_types(G, stream, ktype, vtype, ascend, n):
    keys, values = sort_case(62 + n, ktype, vtype, n)
    order = stable_order(keys, ascend)
    dk, dv = G.to_device(keys), G.to_device(values)
    G.case_sort_by_key_any(dk, dv, ascend, stream)
    assert np.array_equal(dk.download(stream).view(np.uint8), keys[order].view(np.uint8))
    assert np.array_equal(dv.download(stream).view(np.uint8), values[order].view(np.uint8))


@pytest.mark.gpu
def test_gpu_sort_by_half_keys_is_refused_like_the_reference(G, stream):
    from mshadow_amd.capi import HipError
    dk, dv = G.to_device(np.ones(8, f16)), G.to_device(np.arange(8, dtype=np.int32))
    with pytest.raises(HipError, match="half_t"):
        G.case_sort_by_key_any(dk, dv, True, stream)
