#!/usr/bin/env python3
"""Writes tests/golden/hotpath_vectors.npz: inputs and expected outputs of every hot-path
operation, computed by the REFERENCE's own CPU code (oracle/_ref/libmshadow_ref.so, built by
oracle/Makefile from the reference headers where they are present). The reference cannot
travel to the GPU machine; these small vectors can. Run from the repository root:

    make -C oracle all && python tests/golden/make_golden.py

Arrays are plain float32 / uint16 / int32 (numpy .npz, no pickling). Inputs come from
numpy's PCG64 with fixed seeds and are stored next to the outputs, so the file does not
depend on any generator."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from checkers import DIVTO, MAX, MIN, MINUSTO, PLUSTO, SAVETO, SUM, Checker, have_ref  # noqa: E402

f32 = np.float32


def main():
    if not have_ref():
        sys.exit("oracle/_ref/libmshadow_ref.so is missing: build it with `make -C oracle all` "
                 "on a machine that has the reference sources")
    R = Checker("ref")
    rng = np.random.default_rng(20240611)
    g = {}

    a, b, c, d = (rng.uniform(-1, 1, (37, 129)).astype(f32) for _ in range(4))
    g.update(map_a=a, map_b=b, map_c=c, map_d=d)
    for name, saver in (("saveto", SAVETO), ("plusto", PLUSTO), ("divto", DIVTO)):
        out = np.full(a.shape, 1.5, f32)
        R.map_fused(out, a, b, c, d, saver)
        g["map_out_" + name] = out

    x = rng.standard_normal((9, 5, 7, 11)).astype(f32)
    g["red_x"] = x
    for rname, red in (("sum", SUM), ("max", MAX), ("min", MIN)):
        o = np.zeros(5, f32)
        R.reduce_keep_highdim(o, x, red, SAVETO, 1.0)
        g["red_highdim_" + rname] = o
        o = np.zeros(11, f32)
        R.reduce_keep_lowest(o, x.reshape(-1, 11), red, SAVETO, 1.0)
        g["red_lowest_" + rname] = o
    o = np.full(5, 2.0, f32)
    R.reduce_keep_highdim(o, x, SUM, MINUSTO, 0.75)
    g["red_highdim_sum_minusto_scaled"] = o
    long_m = rng.standard_normal((5000, 24)).astype(f32)
    g["red_long"] = long_m
    o = np.zeros(24, f32)
    R.reduce_keep_lowest(o, long_m, SUM, SAVETO, 1.0)
    g["red_long_lowest_sum"] = o

    logits = (rng.standard_normal((6, 3000)) * 3).astype(f32)
    prob = np.empty_like(logits)
    R.softmax(prob, logits)
    label = np.array([0, 2999, 17, -3, 5000, 1234.9], f32)
    grad = np.empty_like(prob)
    R.softmax_grad(grad, prob, label)
    g.update(sm_logits=logits, sm_prob=prob, sm_label=label, sm_grad=grad)
    # the serial float sum of non-negative terms (the softmax row-sum stage on its own)
    terms = np.exp(logits - logits.max(axis=1, keepdims=True)).astype(f32)
    sums = np.zeros(6, f32)
    R.reduce_keep_highdim(sums, terms.reshape(1, 6, 1, 3000), SUM, SAVETO, 1.0)
    g.update(rowsum_terms=terms, rowsum_sums=sums)

    img = np.round(rng.uniform(-1, 1, (3, 4, 23, 17)) * 8).astype(f32) / 8  # duplicates on purpose
    g["pool_x"] = img
    for rname, red in (("max", MAX), ("sum", SUM), ("min", MIN)):
        p = np.empty((3, 4, 11, 6), f32)
        R.pool(p, img, 3, 2, 2, 3, red)
        gr = rng.standard_normal(p.shape).astype(f32)
        u = np.empty_like(img)
        R.unpool(u, img, p, gr, 3, 2, 2, 3, red)
        g["pool_out_" + rname] = p
        g["unpool_grad_" + rname] = gr
        g["unpool_out_" + rname] = u

    im = rng.uniform(-1, 1, (2, 3, 9, 8)).astype(f32)
    imh = R.float2half(im)
    g.update(patch_img_f32=im, patch_img_f16=imh)
    cfgs = {"k3s1d1p1": (3, 3, 1, 1, 1, 1, 1, 1), "k3x2s2x1p0x2": (3, 2, 2, 1, 1, 1, 0, 2),
            "k2x3s1x2d2p1x0": (2, 3, 1, 2, 2, 2, 1, 0)}
    for name, cfg in cfgs.items():
        shape = Checker.col_shape(2, 3, 9, 8, *cfg)
        col = np.empty(shape, f32)
        R.im2col(col, im, *cfg)
        colh = np.empty(shape, np.uint16)
        R.im2col(colh, imh, *cfg)
        cin = rng.standard_normal(shape).astype(f32)
        cinh = R.float2half(cin * 3)
        back = np.empty_like(im)
        R.col2im(back, cin, *cfg)
        backh = np.empty_like(imh)
        R.col2im(backh, cinh, *cfg)
        g["patch_cfg_" + name] = np.array(cfg, np.int32)
        g["im2col_f32_" + name] = col
        g["im2col_f16_" + name] = colh
        g["col2im_in_f32_" + name] = cin
        g["col2im_in_f16_" + name] = cinh
        g["col2im_out_f32_" + name] = back
        g["col2im_out_f16_" + name] = backh

    fl = np.concatenate([rng.standard_normal(2000).astype(f32) * f32(100),
                         np.array([0, -0.0, 65504, 65520, 65536, 1e-8, 6e-8, 6.1e-5, np.inf,
                                   -np.inf, 2049, 2051, 1 + 2 ** -11, 1 + 3 * 2 ** -11], f32)])
    g.update(half_in=fl, half_bits=R.float2half(fl),
             half_back=R.half2float(np.arange(65536, dtype=np.uint16)))

    out = os.path.join(HERE, "hotpath_vectors.npz")
    np.savez_compressed(out, **g)
    print(f"wrote {out}: {len(g)} arrays, {os.path.getsize(out)} bytes")


if __name__ == "__main__":
    main()
