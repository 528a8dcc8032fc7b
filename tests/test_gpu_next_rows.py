"""GPU parity for the rows next to the hot path - SmoothSoftmaxGrad / ignore_label gradients,
3-D softmax and its gradients, AddTakeGrad, AddTakeGradLargeBatch, IndexFill, SortByKey /
VectorizedSort - through the C ABI and through the C++ functions, against the oracle. Bit for bit everywhere except the
3-D softmax forward (relative 1e-5: device exponential)."""
import ctypes

import numpy as np
import pytest

from checkers import GRAD_IGNORE, GRAD_SMOOTH, Checker
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
def O():
    return Checker("orc")


@pytest.mark.parametrize("shape,pad", [((64, 32000), 0), ((9, 1001), 0), ((9, 1000), 4), ((5, 7), 1)])
@pytest.mark.parametrize("flags", [GRAD_SMOOTH, GRAD_IGNORE, GRAD_SMOOTH | GRAD_IGNORE])
def test_grad_family_2d(G, O, shape, pad, flags):
    rng = np.random.default_rng(5)
    p = rng.uniform(0, 1, shape).astype(f32)
    label = rng.integers(0, shape[1], shape[0]).astype(f32)
    label[1], label[2] = shape[1] + 5, -3.0
    ignore = float(label[3])
    want = np.empty(shape, f32)
    O.softmax_grad_ex(want, p, label, flags, ignore, 0.1)
    for route in ("abi", "expr"):
        dst = G.buffer(shape, f32, pad)
        args = (dst, G.to_device(p, pad), G.to_device(label), flags, ignore, 0.1)
        (G.softmax_grad_ex if route == "abi" else G.case_grad_family)(*args)
        assert_bits_equal(dst.download(), want, f"grad flags={flags} {shape} {route}")


@pytest.mark.parametrize("shape,pad", [((7, 19, 33), 0), ((3, 5, 1), 2), ((2, 1000, 70), 1), ((64, 21, 257), 0),
                                       ((4, 21, 64), 0), ((3, 40, 128), 4), ((2, 8, 12), 0)])
def test_softmax3d_and_grads(G, O, shape, pad):
    rng = np.random.default_rng(6)
    x = (rng.standard_normal(shape) * 3).astype(f32)
    want = np.empty(shape, f32)
    O.softmax3d(want, x)
    for route in ("abi", "expr"):
        dst = G.buffer(shape, f32, pad)
        (G.softmax3d if route == "abi" else G.case_softmax3d)(dst, G.to_device(x, pad))
        got = dst.download()
        rel = np.abs(got.astype(np.float64) - want) / np.maximum(want, np.finfo(f32).tiny)
        assert float(rel[want > 0].max()) <= 1e-5, route
    d0, d1, d2 = shape
    label = rng.integers(-1, d1 + 1, (d0, d2)).astype(f32)
    for flags in range(4):
        wantg = np.empty(shape, f32)
        O.softmax3d_grad(wantg, want, label, flags, 2.0, 0.25)
        for route in ("abi", "expr"):
            dst = G.buffer(shape, f32, pad)
            args = (dst, G.to_device(want, pad), G.to_device(label, pad), flags, 2.0, 0.25)
            (G.softmax3d_grad if route == "abi" else G.case_grad_family)(*args)
            assert_bits_equal(dst.download(), wantg, f"3-D grad flags={flags} {shape} {route}")


@pytest.mark.parametrize("k,n,cols,pad", [(50, 300, 21, 0), (7, 1000, 130, 3), (1000, 64, 5, 0), (3, 1, 1, 0)])
@pytest.mark.parametrize("dtype", [np.int32, np.float32])
def test_rows_by_index(G, O, k, n, cols, pad, dtype):
    rng = np.random.default_rng(8)
    src = rng.standard_normal((n, cols)).astype(f32)
    start = rng.standard_normal((k, cols)).astype(f32)
    idx = rng.integers(-3, k + 3, n).astype(dtype)
    want = O.add_take_grad(start.copy(), idx, src)
    dst = G.to_device(start, pad)
    G.add_take_grad(dst, G.to_device(idx), G.to_device(src, pad))
    assert_bits_equal(dst.download(), want, "AddTakeGrad")

    inside = np.clip(idx, 0, k - 1).astype(dtype)
    order = np.argsort(inside, kind="stable").astype(dtype)
    srt = inside[order.astype(int)].astype(dtype)
    want = O.add_take_grad_large_batch(start.copy(), srt, order, src)
    dst = G.to_device(start, pad)
    G.add_take_grad_large_batch(dst, G.to_device(srt), G.to_device(order), G.to_device(src, pad))
    assert_bits_equal(dst.download(), want, "AddTakeGradLargeBatch")

    want = O.index_fill(start.copy(), inside, src)
    dst = G.to_device(start, pad)
    G.index_fill(dst, G.to_device(inside), G.to_device(src, pad))
    assert_bits_equal(dst.download(), want, "IndexFill")

    if dtype == np.int32:  # the C++ functions
        for op, srt_arg, idx_arg, fn in ((0, None, idx, O.add_take_grad),
                                         (2, None, inside, O.index_fill)):
            want = fn(start.copy(), idx_arg, src)
            dst = G.to_device(start, pad)
            G.case_rows_by_index(op, dst, None, G.to_device(idx_arg), G.to_device(src, pad))
            assert_bits_equal(dst.download(), want, f"C++ route op {op}")
        want = O.add_take_grad_large_batch(start.copy(), srt, order, src)
        dst = G.to_device(start, pad)
        G.case_rows_by_index(1, dst, G.to_device(srt), G.to_device(order), G.to_device(src, pad))
        assert_bits_equal(dst.download(), want, "C++ route op 1")


def test_many_duplicates_keep_index_order(G, O):
    """every entry names one of two rows: 5000 ordered float additions per row"""
    rng = np.random.default_rng(9)
    n, cols = 10000, 70
    src = rng.standard_normal((n, cols)).astype(f32)
    idx = rng.integers(0, 2, n).astype(np.int32)
    start = np.zeros((2, cols), f32)
    want = O.add_take_grad(start.copy(), idx, src)
    dst = G.to_device(start)
    G.add_take_grad(dst, G.to_device(idx), G.to_device(src))
    assert_bits_equal(dst.download(), want, "ordered accumulation")


# ---- SortByKey / VectorizedSort
def _sort_inputs(kind, n, seed):
    rng = np.random.default_rng(seed)
    if kind == "f32":
        keys = (rng.integers(-40, 41, n).astype(f32) * f32(0.25)) if n < 5000 else \
            rng.standard_normal(n).astype(f32)
        keys[rng.random(n) < 0.05] = f32(-0.0)
        keys[rng.random(n) < 0.05] = f32(0.0)
        if n > 8:
            keys[:4] = [np.inf, -np.inf, np.finfo(f32).max, np.finfo(f32).tiny / 4]
        values = np.arange(n, dtype=np.int32)
    else:
        keys = rng.integers(-50, 51, n).astype(np.int32) if n < 5000 else \
            rng.integers(-2**31, 2**31, n, dtype=np.int64).astype(np.int32)
        if n > 8:
            keys[:2] = [np.iinfo(np.int32).min, np.iinfo(np.int32).max]
        values = rng.standard_normal(n).astype(f32)
    return keys, values


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["f32", "i32"])
@pytest.mark.parametrize("n", [1, 2, 255, 1000, 65537, 1 << 20])
@pytest.mark.parametrize("ascend", [True, False])
def test_sort_by_key(G, O, kind, n, ascend):
    keys, values = _sort_inputs(kind, n, 3 + n)
    want_k, want_v = O.sort_by_key(keys.copy(), values.copy(), ascend)
    for route in ("abi", "header"):
        dk, dv = G.to_device(keys), G.to_device(values)
        if route == "abi":
            G.sort_by_key(dk, dv, ascend)
        else:
            G.case_sort_by_key(0, dk, dv, ascend)
        assert np.array_equal(dk.download().view(np.uint32), want_k.view(np.uint32)), route
        assert np.array_equal(dv.download().view(np.uint32), want_v.view(np.uint32)), route


@pytest.mark.gpu
def test_sort_by_key_unsigned_and_empty(G):
    rng = np.random.default_rng(8)
    keys = rng.integers(0, 2**32, 5000, dtype=np.int64).astype(np.uint32)
    values = np.arange(5000, dtype=np.int32)
    dk, dv = G.to_device(keys), G.to_device(values)
    G.sort_by_key(dk, dv, False)
    order = np.argsort(-keys.astype(np.int64), kind="stable")
    assert np.array_equal(dk.download(), keys[order]) and np.array_equal(dv.download(), values[order])
    need = ctypes.c_size_t(7)
    G.check(G.dll.mshadow_hip_sort_by_key_workspace(0, ctypes.byref(need)))
    assert need.value == 0
    G.check(G.dll.mshadow_hip_sort_by_key_32(None, 0, None, 0, 1, None, 0, None))
    assert G.dll.mshadow_hip_sort_by_key_32(dk.ptr, 0, dv.ptr, 5000, 1, dk.ptr, 16, None) != 0


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["f32", "i32"])
def test_vectorized_sort(G, O, kind):
    n = 30000
    keys, _ = _sort_inputs(kind, n, 21)
    seg = np.sort(np.random.default_rng(4).integers(0, 300, n)).astype(np.int32)
    want_v, want_s = O.vectorized_sort(keys.copy(), seg.copy())
    dv, ds = G.to_device(keys), G.to_device(seg)
    G.case_sort_by_key(1, dv, ds)
    assert np.array_equal(dv.download().view(np.uint32), want_v.view(np.uint32))
    assert np.array_equal(ds.download(), want_s)
