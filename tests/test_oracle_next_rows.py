"""CPU checks of the oracle for the rows next to the hot path: the rest of the softmax family
(smooth / ignore_label gradients, 3-D softmax and its gradients) and the row scatter / gather
functions (AddTakeGrad, AddTakeGradLargeBatch, IndexFill; mshadow/tensor_cpu-inl.h:304-528).
The reference's own tests do not cover these functions, so they are pinned by closed forms
and brute force here, and bit for bit against the reference build where it is present."""
import numpy as np
import pytest

from checkers import GRAD_IGNORE, GRAD_SMOOTH, Checker, have_ref

f32 = np.float32


def _rng():
    return np.random.default_rng(77)


@pytest.mark.parametrize("flags", [0, GRAD_SMOOTH, GRAD_IGNORE, GRAD_SMOOTH | GRAD_IGNORE])
def test_grad_family_closed_form(orc, flags):
    rng = _rng()
    rows, cols, alpha, ignore = 9, 13, f32(0.1), f32(4)
    p = rng.uniform(0, 1, (rows, cols)).astype(f32)
    label = np.array([0, 12, 4, 4, 7, -2, 13, 3, 4], f32)   # 4 = ignored, -2 / 13 out of range
    out = np.empty_like(p)
    orc.softmax_grad_ex(out, p, label, flags, float(ignore), float(alpha))
    want = p.copy()
    if flags & GRAD_SMOOTH:
        want = (want - f32(alpha / f32(cols - 1))).astype(f32)
    for y, k in enumerate(label.astype(int)):
        if 0 <= k < cols:
            want[y, k] = p[y, k] - f32(1)
            if flags & GRAD_SMOOTH:
                want[y, k] = want[y, k] + alpha
        if (flags & GRAD_IGNORE) and k == int(ignore):
            want[y, :] = 0
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    if flags == 0:
        plain = np.empty_like(p)
        orc.softmax_grad(plain, p, label)
        assert np.array_equal(plain, out)


def test_softmax3d_is_columnwise_softmax(orc):
    rng = _rng()
    x = (rng.standard_normal((5, 17, 23)) * 3).astype(f32)
    out = np.empty_like(x)
    orc.softmax3d(out, x)
    # the same numbers as the 2-D softmax of the rows (y, n) laid out along x
    flat = np.ascontiguousarray(x.transpose(0, 2, 1)).reshape(-1, 17)
    want = np.empty_like(flat)
    orc.softmax(want, flat)
    assert np.array_equal(out.transpose(0, 2, 1).reshape(-1, 17), want)
    assert np.allclose(out.sum(axis=1), 1.0, atol=1e-6)
    uni = np.full((2, 8, 3), 0.25, f32)
    o2 = np.empty_like(uni)
    orc.softmax3d(o2, uni)
    assert np.all(o2 == f32(0.125))


@pytest.mark.parametrize("flags", [0, GRAD_SMOOTH, GRAD_IGNORE, GRAD_SMOOTH | GRAD_IGNORE])
def test_softmax3d_grad_matches_2d_family(orc, flags):
    rng = _rng()
    d0, d1, d2 = 4, 11, 6
    p = rng.uniform(0, 1, (d0, d1, d2)).astype(f32)
    label = rng.integers(-1, d1 + 1, (d0, d2)).astype(f32)
    out = np.empty_like(p)
    orc.softmax3d_grad(out, p, label, flags, 3.0, 0.2)
    flat = np.ascontiguousarray(p.transpose(0, 2, 1)).reshape(-1, d1)
    want = np.empty_like(flat)
    orc.softmax_grad_ex(want, flat, label.reshape(-1), flags, 3.0, 0.2)
    assert np.array_equal(out.transpose(0, 2, 1).reshape(-1, d1), want)


@pytest.mark.parametrize("dtype", [np.int32, np.float32])
def test_take_and_fill_brute_force(orc, dtype):
    rng = _rng()
    k, n, cols = 7, 40, 5
    src = rng.standard_normal((n, cols)).astype(f32)
    idx = rng.integers(-2, k + 2, n).astype(dtype)          # clamped by AddTakeGrad
    dst = rng.standard_normal((k, cols)).astype(f32)
    want = dst.copy()
    for y in range(n):
        j = min(max(int(idx[y]), 0), k - 1)
        want[j] = want[j] + src[y]                           # float32 adds in index order
    got = orc.add_take_grad(dst.copy(), idx, src)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))

    inside = rng.integers(0, k, n).astype(dtype)
    order = np.argsort(inside, kind="stable").astype(dtype)
    sorted_rows = inside[order.astype(int)].astype(dtype)
    want = dst.copy()
    for y in range(n):
        want[int(sorted_rows[y])] = want[int(sorted_rows[y])] + src[int(order[y])]
    got = orc.add_take_grad_large_batch(dst.copy(), sorted_rows, order, src)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the sorted form adds the same rows to the same places in the same order
    assert np.array_equal(got, orc.add_take_grad(dst.copy(), inside, src))

    want = dst.copy()
    for y in range(n):
        want[int(inside[y])] = src[y]                        # the last writer wins
    got = orc.index_fill(dst.copy(), inside, src)
    assert np.array_equal(got, want)


@pytest.mark.skipif(not have_ref(), reason="reference build absent")
def test_oracle_equals_reference_build(orc, ref):
    rng = _rng()
    p = rng.uniform(0, 1, (33, 257)).astype(f32)
    label = rng.integers(-3, 260, 33).astype(f32)
    for flags in range(4):
        a, b = np.empty_like(p), np.empty_like(p)
        orc.softmax_grad_ex(a, p, label, flags, float(label[5]), 0.3)
        ref.softmax_grad_ex(b, p, label, flags, float(label[5]), 0.3)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), flags
    x = (rng.standard_normal((6, 40, 19)) * 3).astype(f32)
    a, b = np.empty_like(x), np.empty_like(x)
    orc.softmax3d(a, x)
    ref.softmax3d(b, x)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    lab = rng.integers(-1, 41, (6, 19)).astype(f32)
    for flags in range(4):
        g1, g2 = np.empty_like(x), np.empty_like(x)
        orc.softmax3d_grad(g1, a, lab, flags, 7.0, 0.05)
        ref.softmax3d_grad(g2, a, lab, flags, 7.0, 0.05)
        assert np.array_equal(g1.view(np.uint32), g2.view(np.uint32)), flags
    for dtype in (np.int32, np.float32):
        src = rng.standard_normal((300, 21)).astype(f32)
        idx = rng.integers(-5, 60, 300).astype(dtype)
        d1 = rng.standard_normal((50, 21)).astype(f32)
        d2 = d1.copy()
        orc.add_take_grad(d1, idx, src)
        ref.add_take_grad(d2, idx, src)
        assert np.array_equal(d1.view(np.uint32), d2.view(np.uint32))
        inside = np.clip(idx, 0, 49).astype(dtype)
        order = np.argsort(inside, kind="stable").astype(dtype)
        srt = inside[order.astype(int)].astype(dtype)
        d1, d2 = d1.copy(), d1.copy()
        orc.add_take_grad_large_batch(d1, srt, order, src)
        ref.add_take_grad_large_batch(d2, srt, order, src)
        assert np.array_equal(d1.view(np.uint32), d2.view(np.uint32))
        orc.index_fill(d1, inside, src)
        ref.index_fill(d2, inside, src)
        assert np.array_equal(d1.view(np.uint32), d2.view(np.uint32))


# ---- SortByKey / VectorizedSort (mshadow/tensor_cpu-inl.h:531-566)
def _sort_inputs(kind, n, seed):
    rng = np.random.default_rng(seed)
    if kind == "f32":
        # few distinct values: long runs of equivalent keys, both zeros among them
        keys = rng.integers(-4, 5, n).astype(f32) * f32(0.5)
        keys[rng.random(n) < 0.1] = f32(-0.0)
        values = np.arange(n, dtype=np.int32)
    else:
        keys = rng.integers(-5, 6, n).astype(np.int32)
        keys[: n // 7] = np.iinfo(np.int32).min
        keys[n // 7: 2 * (n // 7)] = np.iinfo(np.int32).max
        rng.shuffle(keys)
        values = np.arange(n, dtype=f32)
    return keys, values


def _stable_order(keys, ascend):
    """positions in the order a stable sort under < (or >) leaves them: equivalent keys (which
    includes +0.0 and -0.0) keep their original order in both directions"""
    ranks = keys.astype(np.float64)
    return np.argsort(ranks if ascend else -ranks, kind="stable")


@pytest.mark.parametrize("kind", ["f32", "i32"])
@pytest.mark.parametrize("n", [0, 1, 2, 17, 1000, 4099])
@pytest.mark.parametrize("ascend", [True, False])
def test_sort_by_key_is_the_stable_permutation(orc, kind, n, ascend):
    keys, values = _sort_inputs(kind, n, 5 + n)
    order = _stable_order(keys, ascend)
    k, v = keys.copy(), values.copy()
    orc.sort_by_key(k, v, ascend)
    assert np.array_equal(k.view(np.uint32), keys[order].view(np.uint32))   # -0.0 stays -0.0
    assert np.array_equal(v, values[order])


def test_vectorized_sort_sorts_inside_segments(orc):
    rng = np.random.default_rng(11)
    seg = np.sort(rng.integers(0, 9, 500)).astype(np.int32)
    vals = rng.standard_normal(500).astype(f32)
    v, s = vals.copy(), seg.copy()
    orc.vectorized_sort(v, s)
    assert np.array_equal(s, seg)
    for g in np.unique(seg):
        assert np.array_equal(v[seg == g], np.sort(vals[seg == g]))


@pytest.mark.skipif(not have_ref(), reason="reference build absent")
@pytest.mark.parametrize("kind", ["f32", "i32"])
@pytest.mark.parametrize("n", [1, 33, 2048, 50001])
@pytest.mark.parametrize("ascend", [True, False])
def test_sort_by_key_matches_reference_build(orc, ref, kind, n, ascend):
    keys, values = _sort_inputs(kind, n, 9 + n)
    ko, vo = orc.sort_by_key(keys.copy(), values.copy(), ascend)
    kr, vr = ref.sort_by_key(keys.copy(), values.copy(), ascend)
    assert np.array_equal(ko.view(np.uint32), kr.view(np.uint32))
    assert np.array_equal(vo.view(np.uint32), vr.view(np.uint32))
    seg = np.sort(np.random.default_rng(n).integers(0, 1 + n // 5, n)).astype(np.int32)
    a, b = orc.vectorized_sort(keys.copy(), seg.copy())
    c, d = ref.vectorized_sort(keys.copy(), seg.copy())
    assert np.array_equal(a.view(np.uint32), c.view(np.uint32)) and np.array_equal(b, d)
