"""mshadow_hip_sort_by_key_32_noalloc (scratch memory inside the library) against
mshadow_hip_sort_by_key_32 (scratch memory from the caller), through the C ABI, bit for bit:
two calls in a row on the same GPU, the second with a smaller input, so what the first call
left in the scratch array is there when the second runs."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

NOALLOC_MAX = 1 << 20


@pytest.fixture(scope="module")
def G():
    import mshadow_amd
    g = mshadow_amd.load_lib()
    assert g.device_count() >= 1, "no GPU visible"
    g.set_device(0)
    return g


def _pairs(kind, n, seed):
    rng = np.random.default_rng(seed)
    if kind == "f32":
        keys = rng.standard_normal(n).astype(np.float32)
        keys[rng.random(n) < 0.1] = np.float32(-0.0)
        keys[rng.random(n) < 0.1] = np.float32(0.0)
        keys[rng.random(n) < 0.2] = np.float32(1.5)  # runs of equal keys: stability shows
    else:
        keys = rng.integers(-1000, 1000, n).astype(np.int32)
    return keys, np.arange(n, dtype=np.int32)


def _both(G, keys, values, ascend):
    wk, wv = G.to_device(keys), G.to_device(values)
    G.sort_by_key(wk, wv, ascend)
    nk, nv = G.to_device(keys), G.to_device(values)
    G.sort_by_key_noalloc(nk, nv, ascend)
    return (wk.download(), wv.download()), (nk.download(), nv.download())


@pytest.mark.parametrize("kind", ["f32", "i32"])
@pytest.mark.parametrize("sizes", [(NOALLOC_MAX, 70001), (65537, 1000), (300, 1)])
def test_noalloc_matches_workspace_entry_twice(G, kind, sizes):
    for call, n in enumerate(sizes):
        for ascend in (True, False):
            keys, values = _pairs(kind, n, 11 * n + call)
            want, got = _both(G, keys, values, ascend)
            assert np.array_equal(got[0].view(np.uint32), want[0].view(np.uint32)), (n, ascend)
            assert np.array_equal(got[1], want[1]), (n, ascend)
            # and the result is a stable sort of the input
            order = np.argsort(keys if ascend else -keys.astype(np.float64), kind="stable")
            assert np.array_equal(got[1], values[order]), (n, ascend)


def test_noalloc_rejects_more_than_the_maximum_and_takes_empty_input(G):
    keys, values = _pairs("i32", 16, 0)
    dk, dv = G.to_device(keys), G.to_device(values)
    rc = G.dll.mshadow_hip_sort_by_key_32_noalloc(dk.ptr, 1, dv.ptr, NOALLOC_MAX + 1, 1, None)
    assert rc != 0
    assert b"MSHADOW_HIP_SORT_NOALLOC_MAX" in G.dll.mshadow_hip_last_error()
    G.check(G.dll.mshadow_hip_sort_by_key_32_noalloc(None, 1, None, 0, 1, None))
    assert np.array_equal(dk.download(), keys)
