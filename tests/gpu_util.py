"""Helpers for the GPU parity tests: seeded inputs, device buffers, bit comparison."""
import numpy as np

f32 = np.float32


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view({4: np.uint32, 2: np.uint16}[a.dtype.itemsize])


def assert_bits_equal(got, want, what=""):
    g, w = bits(got), bits(want)
    if not np.array_equal(g, w):
        bad = np.flatnonzero(g.ravel() != w.ravel())
        i = bad[0]
        raise AssertionError(
            f"{what}: {bad.size} of {g.size} elements differ; first at flat index {i}: "
            f"got {got.ravel()[i]!r} want {want.ravel()[i]!r}")


def uniform(seed, shape):
    return np.random.default_rng(seed).uniform(-1, 1, shape).astype(f32)


def normal(seed, shape, sigma=1.0):
    return (np.random.default_rng(seed).standard_normal(shape, dtype=f32) * f32(sigma)).astype(f32)


def host_padded(arr, pad):
    """Copy of arr in a host buffer whose rows carry `pad` extra elements (for the oracle)."""
    full = np.empty(arr.shape[:-1] + (arr.shape[-1] + pad,), dtype=arr.dtype)
    view = full[..., : arr.shape[-1]]
    view[...] = arr
    return view
