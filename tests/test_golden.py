"""The committed vectors of tests/golden/hotpath_vectors.npz - written by the reference's own
CPU code, see tests/golden/make_golden.py - against the C oracle (CPU) and against the HIP
path through the C ABI (GPU). Bit for bit everywhere except the softmax forward, whose
exponential is libm's on the host (relative 1e-5 there, as everywhere in this repository)."""
import os

import numpy as np
import pytest

from checkers import DIVTO, MAX, MIN, MINUSTO, PLUSTO, SAVETO, SUM, Checker
from gpu_util import assert_bits_equal, f32

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                            "hotpath_vectors.npz"))
REDUCERS = (("sum", SUM), ("max", MAX), ("min", MIN))
PATCH_CFGS = [k[len("patch_cfg_"):] for k in GOLD.files if k.startswith("patch_cfg_")]


# ------------------------------------------------------------------ oracle (CPU)
def test_oracle_map(orc):
    a, b, c, d = (GOLD["map_" + k] for k in "abcd")
    for name, saver in (("saveto", SAVETO), ("plusto", PLUSTO), ("divto", DIVTO)):
        out = np.full(a.shape, 1.5, f32)
        orc.map_fused(out, a, b, c, d, saver)
        assert_bits_equal(out, GOLD["map_out_" + name], name)


def test_oracle_reductions(orc):
    x = GOLD["red_x"]
    for rname, red in REDUCERS:
        o = np.zeros(5, f32)
        orc.reduce_keep_highdim(o, x, red, SAVETO, 1.0)
        assert_bits_equal(o, GOLD["red_highdim_" + rname], rname)
        o = np.zeros(11, f32)
        orc.reduce_keep_lowest(o, x.reshape(-1, 11), red, SAVETO, 1.0)
        assert_bits_equal(o, GOLD["red_lowest_" + rname], rname)
    o = np.full(5, 2.0, f32)
    orc.reduce_keep_highdim(o, x, SUM, MINUSTO, 0.75)
    assert_bits_equal(o, GOLD["red_highdim_sum_minusto_scaled"], "minusto")
    o = np.zeros(24, f32)
    orc.reduce_keep_lowest(o, GOLD["red_long"], SUM, SAVETO, 1.0)
    assert_bits_equal(o, GOLD["red_long_lowest_sum"], "long columns")


def test_oracle_softmax(orc):
    prob = np.empty_like(GOLD["sm_logits"])
    orc.softmax(prob, GOLD["sm_logits"])
    assert_bits_equal(prob, GOLD["sm_prob"], "softmax (same libm on this host)")
    grad = np.empty_like(prob)
    orc.softmax_grad(grad, GOLD["sm_prob"], GOLD["sm_label"])
    assert_bits_equal(grad, GOLD["sm_grad"], "softmax grad")


def test_oracle_pool_unpool(orc):
    x = GOLD["pool_x"]
    for rname, red in REDUCERS:
        p = np.empty(GOLD["pool_out_" + rname].shape, f32)
        orc.pool(p, x, 3, 2, 2, 3, red)
        assert_bits_equal(p, GOLD["pool_out_" + rname], rname)
        u = np.empty_like(x)
        orc.unpool(u, x, p, GOLD["unpool_grad_" + rname], 3, 2, 2, 3, red)
        assert_bits_equal(u, GOLD["unpool_out_" + rname], rname)


@pytest.mark.parametrize("name", PATCH_CFGS)
def test_oracle_patches(orc, name):
    cfg = [int(v) for v in GOLD["patch_cfg_" + name]]
    for t, img in (("f32", GOLD["patch_img_f32"]), ("f16", GOLD["patch_img_f16"])):
        col = np.empty_like(GOLD[f"im2col_{t}_{name}"])
        orc.im2col(col, img, *cfg)
        assert np.array_equal(col.view(np.uint8), GOLD[f"im2col_{t}_{name}"].view(np.uint8))
        back = np.empty_like(img)
        orc.col2im(back, GOLD[f"col2im_in_{t}_{name}"], *cfg)
        assert np.array_equal(back.view(np.uint8), GOLD[f"col2im_out_{t}_{name}"].view(np.uint8))


def test_oracle_half(orc):
    assert np.array_equal(orc.float2half(GOLD["half_in"]), GOLD["half_bits"])
    back = orc.half2float(np.arange(65536, dtype=np.uint16))
    assert np.array_equal(back.view(np.uint32), GOLD["half_back"].view(np.uint32))


# ------------------------------------------------------------------ HIP path (GPU)
@pytest.fixture(scope="module")
def G():
    import mshadow_amd
    g = mshadow_amd.load_cases()
    assert g.device_count() >= 1, "no GPU visible"
    g.set_device(0)
    return g


@pytest.mark.gpu
def test_gpu_map(G):
    dev = [G.to_device(GOLD["map_" + k], pad) for k, pad in zip("abcd", (0, 3, 0, 1))]
    for name, saver in (("saveto", SAVETO), ("plusto", PLUSTO), ("divto", DIVTO)):
        out = G.to_device(np.full(GOLD["map_a"].shape, 1.5, f32))
        G.case_map_fused(out, *dev, saver, None)
        assert_bits_equal(out.download(), GOLD["map_out_" + name], name)


@pytest.mark.gpu
def test_gpu_reductions(G):
    x = GOLD["red_x"]
    dx = G.to_device(x)
    d2 = G.to_device(x.reshape(-1, 11))
    for rname, red in REDUCERS:
        o = G.buffer((5,), f32)
        G.reduce_keep_highdim(o, dx, red, SAVETO, 1.0)
        assert_bits_equal(o.download(), GOLD["red_highdim_" + rname], rname)
        o = G.buffer((11,), f32)
        G.reduce_keep_lowest(o, d2, red, SAVETO, 1.0)
        assert_bits_equal(o.download(), GOLD["red_lowest_" + rname], rname)
    o = G.to_device(np.full(5, 2.0, f32))
    G.reduce_keep_highdim(o, dx, SUM, MINUSTO, 0.75)
    assert_bits_equal(o.download(), GOLD["red_highdim_sum_minusto_scaled"], "minusto")
    o = G.buffer((24,), f32)
    G.reduce_keep_lowest(o, G.to_device(GOLD["red_long"]), SUM, SAVETO, 1.0)
    assert_bits_equal(o.download(), GOLD["red_long_lowest_sum"], "long columns (direct-to-LDS kernel)")


@pytest.mark.gpu
def test_gpu_softmax(G):
    want = GOLD["sm_prob"]
    out = G.buffer(want.shape, f32)
    G.softmax(out, G.to_device(GOLD["sm_logits"]))
    got = out.download()
    rel = np.abs(got.astype(np.float64) - want) / np.maximum(want, np.finfo(f32).tiny)
    assert float(rel[want > 0].max()) <= 1e-5
    grad = G.buffer(want.shape, f32)
    G.softmax_grad(grad, G.to_device(want), G.to_device(GOLD["sm_label"]))
    assert_bits_equal(grad.download(), GOLD["sm_grad"], "softmax grad")
    sums = G.buffer((want.shape[0],), f32)
    G.softmax_rowsum(sums, G.to_device(GOLD["rowsum_terms"]))
    assert_bits_equal(sums.download(), GOLD["rowsum_sums"], "row sum in the reference's order")


@pytest.mark.gpu
def test_gpu_pool_unpool(G):
    x = GOLD["pool_x"]
    dx = G.to_device(x)
    for rname, red in REDUCERS:
        p = G.buffer(GOLD["pool_out_" + rname].shape, f32)
        G.pool(p, dx, 3, 2, 2, 3, red)
        assert_bits_equal(p.download(), GOLD["pool_out_" + rname], rname)
        u = G.buffer(x.shape, f32)
        G.unpool(u, dx, p, G.to_device(GOLD["unpool_grad_" + rname]), 3, 2, 2, 3, red)
        assert_bits_equal(u.download(), GOLD["unpool_out_" + rname], rname)


@pytest.mark.gpu
@pytest.mark.parametrize("name", PATCH_CFGS)
def test_gpu_patches(G, name):
    cfg = [int(v) for v in GOLD["patch_cfg_" + name]]
    for t, img in (("f32", GOLD["patch_img_f32"]), ("f16", GOLD["patch_img_f16"])):
        want = GOLD[f"im2col_{t}_{name}"]
        col = G.buffer(want.shape, want.dtype)
        G.im2col(col, G.to_device(img), *cfg)
        assert np.array_equal(col.download().view(np.uint8), want.view(np.uint8)), f"im2col {t}"
        want = GOLD[f"col2im_out_{t}_{name}"]
        back = G.buffer(img.shape, img.dtype)
        G.col2im(back, G.to_device(GOLD[f"col2im_in_{t}_{name}"]), *cfg)
        assert np.array_equal(back.download().view(np.uint8), want.view(np.uint8)), f"col2im {t}"
