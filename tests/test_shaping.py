"""broadcast<1> / repmat / reshape / swapaxis / mirror / upsampling_nearest / broadcast_scalar:
the expressions of mshadow_case_shaping_f32 (the convnet's bias-add and layout-change idioms,
guide/neuralnet/convnet.cu:88,96,99,155,176 of the reference) against numpy, on the reference
build (CPU, where present) and on the GPU through the generic expression kernel. Pure data
movement plus one exact operation per element: bit for bit."""
import numpy as np
import pytest

from checkers import Checker, have_ref

f32 = np.float32
SHAPES = [(2, 3, 4, 5), (5, 1, 7, 3), (3, 8, 2, 64), (1, 2, 1, 1)]


def numpy_shaping(op, a, v):
    n, c, h, w = a.shape
    if op == 0:
        return a + v[:c].reshape(1, c, 1, 1)
    if op == 1:
        return (a.reshape(n * c * h, w) + v[:w]).astype(f32)
    if op == 2:   # input read as (n, c, h, w), result (c, n, h, w)
        return a.transpose(1, 0, 2, 3)
    if op == 3:
        return a.transpose(1, 0, 2, 3).reshape(c, n * h * w)
    if op == 4:
        return a.transpose(0, 3, 2, 1)
    if op == 5:
        return a.transpose(0, 2, 1, 3)
    if op == 6:
        return a[..., ::-1]
    if op == 7:
        return a.repeat(2, axis=2).repeat(2, axis=3)
    if op == 8:
        return (v[0] * a).astype(f32)
    return (v[: a.size] * f32(2)).reshape(n * c, h * w)


def _inputs(shape):
    rng = np.random.default_rng(sum(shape))
    a = rng.standard_normal(shape).astype(f32)
    v = rng.standard_normal(max(a.size, 8)).astype(f32)
    return a, v


@pytest.mark.skipif(not have_ref(), reason="reference build absent")
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("op", range(10))
def test_reference_build_matches_numpy(ref, shape, op):
    a, v = _inputs(shape)
    want = np.ascontiguousarray(numpy_shaping(op, a, v), dtype=f32)
    out = np.empty(want.shape, f32)
    ref.shaping(op, out, a, v, *shape)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", SHAPES + [(16, 32, 28, 28)])
@pytest.mark.parametrize("op", range(10))
def test_gpu_matches_numpy(shape, op):
    import mshadow_amd
    G = mshadow_amd.load_cases()
    G.set_device(0)
    a, v = _inputs(shape)
    want = np.ascontiguousarray(numpy_shaping(op, a, v), dtype=f32)
    out = G.buffer(want.shape, f32)
    G.case_shaping(op, out, G.to_device(a), G.to_device(v), *shape)
    got = out.download()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (op, shape)
