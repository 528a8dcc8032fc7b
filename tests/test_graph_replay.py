"""The hot path recorded into a HIP graph and replayed: every replay must give, bit for bit, what
the same launches give when queued one by one. The replays are separated by launches of the
program's own (a kernel that overwrites the outputs) and by synchronisations, so a node that only
works the first time would show."""
import numpy as np
import pytest

from gpu_util import assert_bits_equal

pytestmark = pytest.mark.gpu
f32 = np.float32


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


def _operands(G, rng, scale):
    n = 4096 // scale
    d = {"A": rng.standard_normal((n, 1024), dtype=f32), "B": rng.standard_normal((n, 1024), dtype=f32),
         "C": rng.standard_normal((n, 1024), dtype=f32), "D": rng.standard_normal((n, 1024), dtype=f32),
         "X2a": rng.standard_normal((64 // scale, 256, 14, 14), dtype=f32),
         "M2b": rng.standard_normal((4096 // scale, 1024), dtype=f32),
         "L": rng.standard_normal((512 // scale, 32000), dtype=f32) * f32(3),
         "X4": rng.standard_normal((16 // scale, 64, 112, 112), dtype=f32),
         # few kept indices: the split reduction with its scratch slot and counters
         "Xfew": rng.standard_normal((40, 8, 48, 48), dtype=f32)}
    dev = {k: G.to_device(v) for k, v in d.items()}
    dev["labels"] = G.to_device(rng.integers(0, 32000, d["L"].shape[0]).astype(f32))
    img = rng.standard_normal((8 // scale, 64, 56, 56)).astype(np.float16).view(np.uint16)
    dev["img"] = G.to_device(img)
    p = d["X4"].shape
    out = {"map": G.buffer(d["A"].shape, f32), "2a": G.buffer((256,), f32), "2b": G.buffer((1024,), f32),
           "few": G.buffer((8,), f32), "p": G.buffer(d["L"].shape, f32), "g": G.buffer(d["L"].shape, f32),
           "pool": G.buffer((p[0], p[1], 55, 55), f32), "unpool": G.buffer(p, f32),
           "col": G.buffer((64 * 9, img.shape[0] * 56 * 56), np.uint16), "img": G.buffer(img.shape, np.uint16)}
    dev["G4"] = G.to_device(rng.standard_normal((p[0], p[1], 55, 55), dtype=f32))
    return dev, out


def _step(G, dev, out, s):
    G.case_map_fused(out["map"], dev["A"], dev["B"], dev["C"], dev["D"], 0, s)
    G.reduce_keep_highdim(out["2a"], dev["X2a"], stream=s)
    G.reduce_keep_highdim(out["few"], dev["Xfew"], stream=s)
    G.reduce_keep_lowest(out["2b"], dev["M2b"], stream=s)
    G.softmax(out["p"], dev["L"], s)
    G.softmax_grad(out["g"], out["p"], dev["labels"], s)
    G.pool(out["pool"], dev["X4"], 3, 3, 2, 2, stream=s)
    G.unpool(out["unpool"], dev["X4"], out["pool"], dev["G4"], 3, 3, 2, 2, stream=s)
    G.im2col(out["col"], dev["img"], 3, 3, 1, 1, 1, 1, 1, 1, s)
    G.col2im(out["img"], out["col"], 3, 3, 1, 1, 1, 1, 1, 1, s)


def _snapshot(out, s):
    return {k: v.download(s).copy() for k, v in out.items()}


def _scribble(G, out, s):
    for v in out.values():
        if v.dtype == np.float32:
            G.fill(v, 7.0, s)


def test_hot_path_replayed_from_a_graph(G, stream):
    rng = np.random.default_rng(90)
    dev, out = _operands(G, rng, 1)
    _step(G, dev, out, stream)           # one by one: the expected results (and every lazy set-up done)
    G.stream_sync(stream)
    want = _snapshot(out, stream)
    _scribble(G, out, stream)
    G.stream_sync(stream)
    G.graph_begin(stream)
    _step(G, dev, out, stream)
    graph = G.graph_end(stream)
    try:
        for replay in range(3):
            G.graph_launch(graph, stream)
            G.stream_sync(stream)
            got = _snapshot(out, stream)
            for k in want:
                assert_bits_equal(got[k], want[k], f"replay {replay}: {k}")
            _scribble(G, out, stream)    # the program's own launches between two replays
            G.stream_sync(stream)
        # two replays queued back to back on the stream
        G.graph_launch(graph, stream)
        G.graph_launch(graph, stream)
        G.stream_sync(stream)
        got = _snapshot(out, stream)
        for k in want:
            assert_bits_equal(got[k], want[k], f"back to back: {k}")
    finally:
        G.graph_destroy(graph)


def test_recording_needs_a_stream_of_its_own(G):
    from mshadow_amd.capi import HipError
    with pytest.raises(HipError):
        G.graph_begin(None)
