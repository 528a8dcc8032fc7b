#!/usr/bin/env python3
"""Benchmark of the mshadow hot path on one MI355X.

A step is one pass of the nine hot-path operations over one batch of synthetic inputs of
the shapes named in BASELINE.json (configs 1-5): fused elementwise map, the two
reduce-to-1D forms, softmax forward and gradient, max-pool and its backward, im2col and
col2im. Inputs are generated once from fixed seeds and are resident in HBM before the
timed region; every operation is queued on one stream through the C ABI (the elementwise
map through the C++ expression API compiled in libmshadow_cases.so).

Output: one JSON line. `value` is the whole-step effective bandwidth: algorithmic bytes
(each tensor counted once) of all nine operations divided by the step time of the timed
region - exactly K steps between two synchronizations, with HIP events only around the
dominant operation (`roofline`: the kernel that takes the largest share of the step, timed
live inside the timed region). `per_op` lists each operation's own figures from a pass of
the same K steps made just before, with an event after every launch (`ms`: the interval
inside a step, a few microseconds of launch gap included) and from launches repeated back to
back over rotating operand sets (`ms_back_to_back`). `ms_per_step_graph_replay` is the step
recorded once into a HIP graph and replayed. `cpu_baseline` times the reference CPU
path (oracle/_ref, the reference's own headers) or, where that library is absent, the C
restatement, on the host cores of the same machine over the same inputs.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
f32 = np.float32


def algorithmic_bytes():
    """Compulsory traffic per operation: every tensor read or written once."""
    e = 4
    return {
        "map_fused": 5 * e * 4096 * 4096,
        "sumall_except_dim1": e * 64 * 256 * 56 * 56 + e * 256,
        "sum_rows": e * 16384 * 4096 + e * 4096,
        "softmax": 2 * e * 8192 * 32000,
        "softmax_grad": 2 * e * 8192 * 32000 + e * 8192,
        "pool_max": e * 128 * 64 * 112 * 112 + e * 128 * 64 * 55 * 55,
        "unpool_max": 2 * e * 128 * 64 * 112 * 112 + 2 * e * 128 * 64 * 55 * 55,
        "im2col_f16": 2 * 32 * 256 * 56 * 56 + 2 * 2304 * 100352,
        "col2im_f16": 2 * 32 * 256 * 56 * 56 + 2 * 2304 * 100352,
        "calib_copy": 2 * e * 4096 * 4096,
        # rows next to the hot path (only with --only; never part of the step)
        "smooth_softmax_grad_ignore": 2 * e * 8192 * 32000 + e * 8192,
        "softmax3d": 2 * e * 256 * 21 * 16384,
        "softmax3d_grad": 2 * e * 256 * 21 * 16384 + e * 256 * 16384,
        "add_take_grad": e * 16384 + 3 * e * 16384 * 512,
        "bias_add_broadcast": 2 * e * 64 * 256 * 56 * 56 + e * 256,
        "swapaxis10_reshape": 2 * e * 64 * 256 * 56 * 56,
        "lrn_scale_chpool5": 2 * e * 64 * 256 * 56 * 56,
        "transpose_nchw_nhwc": 2 * e * 64 * 256 * 56 * 56,
        "sort_by_key_f32": 4 * e * (1 << 24),
        # what plain streaming reaches on this machine: a copy and a fill of 8192x32000 floats
        "random_uniform": e * 8192 * 32000,
        "random_normal": e * 8192 * 32000,
        "ceiling_copy": 2 * e * 8192 * 32000,
        "ceiling_fill": e * 8192 * 32000,
        # Copy(Tensor<gpu>, Tensor<gpu>): dense rows; rows of 32000 floats at a pitch of 32064; rows
        # of 31990 floats at a pitch of 32000 (what AllocSpace gives them with padding on)
        "copy_d2d": 2 * e * 8192 * 32000,
        "copy_d2d_pitched": 2 * e * 8192 * 32000,
        "copy_d2d_ragged": 2 * e * 8192 * 31990,
        "dot_f32_4096": 3 * e * 4096 * 4096,
        "dot_f16_8192": 3 * 2 * 8192 * 8192,
        # the same shapes on half_t tensors through the element-type-generic header paths
        "softmax_f16": 2 * 2 * 8192 * 32000,
        "softmax_grad_f16": 2 * 2 * 8192 * 32000 + 2 * 8192,
        "sum_rows_f16": 2 * 16384 * 4096 + 2 * 4096,
        "sumall_except_dim1_f16": 2 * 64 * 256 * 56 * 56 + 2 * 256,
        # sumall_except_dim<1> where few indices are kept: (64,64,112,112) and (256,16,112,112)
        "sumall_except_dim1_64_kept": e * 64 * 64 * 112 * 112 + e * 64,
        "sumall_except_dim1_16_kept": e * 256 * 16 * 112 * 112 + e * 16,
    }


def work_elements():
    return {
        "map_fused": 4096 * 4096, "sumall_except_dim1": 64 * 256 * 56 * 56,
        "sum_rows": 16384 * 4096, "softmax": 8192 * 32000, "softmax_grad": 8192 * 32000,
        "pool_max": 128 * 64 * 55 * 55, "unpool_max": 128 * 64 * 112 * 112,
        "im2col_f16": 2304 * 100352, "col2im_f16": 2304 * 100352, "calib_copy": 4096 * 4096,
        "smooth_softmax_grad_ignore": 8192 * 32000, "softmax3d": 256 * 21 * 16384,
        "softmax3d_grad": 256 * 21 * 16384, "add_take_grad": 16384 * 512,
        "bias_add_broadcast": 64 * 256 * 56 * 56, "swapaxis10_reshape": 64 * 256 * 56 * 56,
        "lrn_scale_chpool5": 64 * 256 * 56 * 56, "transpose_nchw_nhwc": 64 * 256 * 56 * 56,
        "sort_by_key_f32": 1 << 24, "dot_f32_4096": 4096 * 4096, "dot_f16_8192": 8192 * 8192,
        "ceiling_copy": 8192 * 32000, "ceiling_fill": 8192 * 32000,
        "copy_d2d": 8192 * 32000, "copy_d2d_pitched": 8192 * 32000, "copy_d2d_ragged": 8192 * 31990,
        "random_uniform": 8192 * 32000, "random_normal": 8192 * 32000,
        "softmax_f16": 8192 * 32000, "softmax_grad_f16": 8192 * 32000,
        "sum_rows_f16": 16384 * 4096, "sumall_except_dim1_f16": 64 * 256 * 56 * 56,
        "sumall_except_dim1_64_kept": 64 * 64 * 112 * 112, "sumall_except_dim1_16_kept": 256 * 16 * 112 * 112,
    }


# multiply-adds count two: the plain library products (rocBLAS), priced against the dense
# matrix-core peaks (fp32 157.3 TFLOP/s, fp16 2500 TFLOP/s)
PRODUCT_FLOPS = {"dot_f32_4096": (2 * 4096 ** 3, 157.3), "dot_f16_8192": (2 * 8192 ** 3, 2500.0)}


# What a kernel that adds in the reference's order can reach at all: sum_rows is one chain of
# 16384 dependent adds per column, 3.9 ns each with every CU busy (bench.py --only ceiling_chain)
# = 64 us, and its loads - 64 bytes of every row per CU, half a cache line per request, at most
# about 128 requests in flight per CU - take 68 us alone (--only ceiling_lds_loads).
ORDER_FAITHFUL = {
    "sum_rows": {"order_faithful_ceiling": 0.52,
                 "ceiling_from": "16384 dependent adds per column x 3.9 ns = 64 us; column-strip loads alone 68 us"},
}

EXTRA_OPS = ("calib_copy", "smooth_softmax_grad_ignore", "softmax3d", "softmax3d_grad", "add_take_grad",
             "bias_add_broadcast", "swapaxis10_reshape", "lrn_scale_chpool5", "transpose_nchw_nhwc",
             "sort_by_key_f32", "dot_f32_4096", "dot_f16_8192", "ceiling_copy", "ceiling_fill",
             "random_uniform", "random_normal", "softmax_f16", "softmax_grad_f16", "sum_rows_f16",
             "sumall_except_dim1_f16", "copy_d2d", "copy_d2d_pitched", "copy_d2d_ragged",
             "sumall_except_dim1_64_kept", "sumall_except_dim1_16_kept")
OPS = [k for k in algorithmic_bytes() if k not in EXTRA_OPS]

# HBM bytes per launch of each operation's kernel come from the committed counter summary
# (two `rocprofv3 --pmc` runs of this script, FETCH_SIZE then WRITE_SIZE, each counter scaled by
# what it reads for the calibration copy of known size; the command is in the file). bench.py
# cannot run the profiler on itself, so `roofline.traffic` is read from that file at run time.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "hotpath_step_all_kernels_hbm_traffic.md")
TRAFFIC_ROW_OF_OP = {
    "map_fused": "map_fused", "sumall_except_dim1": "ReduceKeepHighDimDmaKernel",
    "sum_rows": "ReduceKeepLowestDmaKernel", "softmax": "SoftmaxRowKernel",
    "softmax_grad": "SoftmaxGradKernel", "pool_max": "PoolKernel", "unpool_max": "UnpoolRows3x3s2Kernel",
    "im2col_f16": "Im2ColRow3DirectKernel", "col2im_f16": "Col2ImHalfRows3x3Kernel",
}


def measured_hbm_bytes(op):
    """bytes one launch of `op`'s kernel moved to and from HBM according to the counter summary
    under profiles/ (columns "HBM read MiB" and "HBM written MiB"), or None"""
    row = TRAFFIC_ROW_OF_OP.get(op)
    try:
        with open(TRAFFIC_PROFILE) as f:
            lines = [l for l in f if l.startswith("|")]
    except OSError:
        return None
    if row is None or not lines:
        return None
    head = [c.strip() for c in lines[0].strip().strip("|").split("|")]
    try:
        rd, wr = head.index("HBM read MiB"), head.index("HBM written MiB")
    except ValueError:
        return None
    for l in lines[2:]:
        cells = [c.strip() for c in l.strip().strip("|").split("|")]
        if cells and cells[0] == row:
            return int(round((float(cells[rd]) + float(cells[wr])) * (1 << 20)))
    return None


def make_inputs(scale=1):
    """Seeded synthetic inputs of the BASELINE shapes (scale > 1 shrinks the leading
    dimension for quick functional runs; the reported benchmark uses scale 1)."""
    def rng(seed):
        return np.random.default_rng(seed)
    s = scale
    d = {}
    d["A"], d["B"], d["C"], d["D"] = (rng(i).uniform(-1, 1, (4096 // s, 4096)).astype(f32)
                                      for i in (1, 2, 3, 4))
    d["X2a"] = rng(5).standard_normal((64 // s, 256, 56, 56), dtype=f32)
    d["M2b"] = rng(6).standard_normal((16384 // s, 4096), dtype=f32)
    d["L"] = rng(7).standard_normal((8192 // s, 32000), dtype=f32) * f32(3)
    d["labels"] = rng(8).integers(0, 32000, 8192 // s).astype(f32)
    d["X4"] = rng(9).uniform(-1, 1, (128 // s, 64, 112, 112)).astype(f32)
    d["G4"] = rng(10).standard_normal((128 // s, 64, 55, 55), dtype=f32)
    return d


def to_half_bits(a):
    """binary16 bit patterns of a float32 array, rounded to nearest even (numpy.float16 rounds
    exactly as half_t's conversion does)"""
    return np.ascontiguousarray(a, dtype=f32).astype(np.float16).view(np.uint16)


def half_inputs(scale=1):
    s = scale
    img = to_half_bits(np.random.default_rng(11).uniform(-1, 1, (32 // s, 256, 56, 56)).astype(f32))
    colshape = (2304, (32 // s) * 56 * 56)
    col = to_half_bits(np.random.default_rng(12).standard_normal(colshape, dtype=f32))
    return img, col


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--scale", type=int, default=1, help="shrink leading dims (functional runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--sets", type=int, default=3, help="complete operand sets the steps take in turn "
                    "(1 = every step on the same buffers; the default keeps a launch from finding "
                    "its operands in the memory-side cache)")
    ap.add_argument("--cpu-reps", type=int, default=30)
    ap.add_argument("--hold", default="", help="comma list of operands that stay those of the first "
                    "set while the others rotate (profiling aid): dimg, out_col, out_unpool, dev.X4, "
                    "dev.G4, ... and nxt for the producer outputs unpool / softmax_grad read")
    ap.add_argument("--only", default="", help="comma list of ops to run (profiling aid); "
                    "softmax_phases, ceiling_chain and ceiling_lds_loads run the probes of "
                    "libmshadow_probe.so instead")
    ap.add_argument("--pattern", default="", help="with --only ceiling_lds_loads: one pattern "
                    "'strip:width:waves' instead of the whole table (for a counter run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; every operation of the path runs at its "
                 "full shape on one MI355X and nothing is sharded (--gpus must be 1)")

    import mshadow_amd
    G = mshadow_amd.load_cases()
    if G.device_count() < 1:
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    G.set_device(0)
    if args.only in ("softmax_phases", "ceiling_chain", "ceiling_lds_loads", "ceiling_seg_loads",
                     "softmax_prefetch_copy", "highdim_split_configs", "staying_waves_copy"):
        return run_probe(G, args.only, args.pattern)
    if args.only == "neighbour_shapes":
        return neighbour_shapes(G)
    props = G.props(0)
    only = [o for o in args.only.split(",") if o] or OPS

    t0 = time.time()
    H = make_inputs(args.scale)
    img_h, col_h = half_inputs(args.scale)
    gen_s = time.time() - t0

    s = G.stream_create()
    def buffer_set():
        """inputs on the device and outputs of their own: one complete set of operands"""
        b = {"dev": {k: G.to_device(v) for k, v in H.items()},
             "dimg": G.to_device(img_h), "dcol_in": G.to_device(col_h),
             "out_map": G.buffer(H["A"].shape, f32), "out_2a": G.buffer((256,), f32),
             "out_2b": G.buffer((4096,), f32), "out_p": G.buffer(H["L"].shape, f32),
             "out_g": G.buffer(H["L"].shape, f32), "out_pool": G.buffer(H["G4"].shape, f32),
             "out_unpool": G.buffer(H["X4"].shape, f32), "out_col": G.buffer(col_h.shape, np.uint16),
             "out_img": G.buffer(img_h.shape, np.uint16)}
        # softmax_grad / unpool consume the outputs of softmax / pool: make them valid first
        G.softmax(b["out_p"], b["dev"]["L"], s)
        G.pool(b["out_pool"], b["dev"]["X4"], 3, 3, 2, 2, stream=s)
        return b

    # Three complete sets of operands, taken in turn step by step, so that no launch finds its
    # input in the 256 MB memory-side cache from the launch before. unpool and softmax_grad read
    # what pool and softmax wrote - from the NEXT set (written two steps ago, same values), not
    # from the launch that has just finished.
    rotate = args.scale == 1 and all(o in OPS for o in only)
    sets = [buffer_set() for _ in range(max(1, args.sets) if rotate else 1)]
    cur = dict(sets[0])     # the set run_op works on
    nxt = dict(sets[1 % len(sets)])   # where unpool / softmax_grad take their producer's output
    dev = cur["dev"]
    out_map, out_g, out_p = cur["out_map"], cur["out_g"], cur["out_p"]

    hold = [x for x in args.hold.split(",") if x]

    def use_set(k):
        cur.update(sets[k % len(sets)])
        nxt.update(sets[(k + 1) % len(sets)])
        if any(x.startswith("dev.") for x in hold):
            cur["dev"] = dict(cur["dev"])
        for x in hold:
            if x == "nxt":
                nxt.update(sets[0])
            elif x.startswith("dev."):
                cur["dev"][x[4:]] = sets[0]["dev"][x[4:]]
            else:
                cur[x] = sets[0][x]

    extra = {}
    if any(o in EXTRA_OPS[1:] for o in only):
        rng = np.random.default_rng(13)
        x3 = (rng.standard_normal((256, 21, 16384), dtype=f32) * f32(3))
        extra["x3"] = G.to_device(x3)
        extra["p3"] = G.buffer(x3.shape, f32)
        extra["g3"] = G.buffer(x3.shape, f32)
        extra["l3"] = G.to_device(rng.integers(0, 21, (256, 16384)).astype(f32))
        extra["emb"] = G.to_device(np.zeros((50000, 512), f32))
        extra["idx"] = G.to_device(rng.integers(0, 50000, 16384).astype(np.int32))
        extra["rows"] = G.to_device(rng.standard_normal((16384, 512), dtype=f32))

    if "sort_by_key_f32" in only:
        import ctypes
        rng = np.random.default_rng(15)
        extra["keys"] = G.to_device(rng.standard_normal(1 << 24, dtype=f32))
        extra["vals"] = G.to_device(np.arange(1 << 24, dtype=np.int32))
        need = ctypes.c_size_t(0)
        G.check(G.dll.mshadow_hip_sort_by_key_workspace(1 << 24, ctypes.byref(need)))
        extra["work"] = G.buffer((need.value,), np.uint8)
        extra["work_bytes"] = need.value
    if any(o in ("bias_add_broadcast", "swapaxis10_reshape", "lrn_scale_chpool5",
                 "transpose_nchw_nhwc") for o in only):
        extra["out4"] = G.buffer(H["X2a"].shape, f32)
        extra["bias"] = G.to_device(np.random.default_rng(14).standard_normal(51380224, dtype=f32)[:256].copy())

    if any(o.endswith("_f16") and o not in OPS for o in only):
        extra["hL"] = G.to_device(to_half_bits(H["L"]))
        extra["hP"] = G.buffer(H["L"].shape, np.uint16)
        extra["hG"] = G.buffer(H["L"].shape, np.uint16)
        # labels a half can hold exactly (integers up to 2048)
        extra["hlab"] = G.to_device(to_half_bits(np.minimum(H["labels"], f32(2048))))
        extra["hM"] = G.to_device(to_half_bits(H["M2b"]))
        extra["hX"] = G.to_device(to_half_bits(H["X2a"]))
        extra["h2b"] = G.buffer((4096,), np.uint16)
        extra["h2a"] = G.buffer((256,), np.uint16)
        G.case_softmax(extra["hP"], extra["hL"], s)

    if any(o.startswith("copy_d2d_") for o in only):
        extra["pitched_src"] = G.buffer(H["L"].shape, f32, pad=64)
        extra["pitched_dst"] = G.buffer(H["L"].shape, f32, pad=64)
    if "dot_f32_4096" in only:   # dst = dot(A, B.T()) through the expression engine
        extra["mm_out"] = G.buffer((4096, 4096), f32)
    if "dot_f16_8192" in only:
        from mshadow_amd import capi
        h = np.random.default_rng(16).standard_normal(8192 * 8192, dtype=f32).astype(np.float16)
        extra["ha"], extra["hb"] = G.to_device(h), G.to_device(h[::-1].copy())
        extra["hc"] = G.buffer((8192 * 8192,), np.float16)
        extra["f16"] = capi.BLAS_F16

    def run_op(name):
        if name == "ceiling_copy":     # dst = (src + 0) / 1 + 0 through the expression kernel
            G.case_map_axpb(out_g, dev["L"], 0.0, 1.0, 0.0, 0, s)
        elif name == "copy_d2d":
            G.case_copy_d2d(out_g, dev["L"], s)
        elif name == "copy_d2d_pitched":
            G.case_copy_d2d(extra["pitched_dst"], extra["pitched_src"], s)
        elif name == "copy_d2d_ragged":
            G.case_copy_d2d(out_g, dev["L"], s, cols=31990)
        elif name == "random_uniform":  # Random<gpu>::SampleUniform over 8192x32000 floats
            G.random_uniform(out_g, 7, 0, 0, -1.0, 1.0, s)
        elif name == "random_normal":   # Random<gpu>::SampleGaussian
            G.random_normal(out_g, 7, 0, 0, 0.0, 1.0, s)
        elif name == "ceiling_fill":   # dst = scalar
            G.fill(out_g, 1.0, s)
        elif name == "softmax_f16":     # Softmax(Tensor<gpu,2,half_t>, ...)
            G.case_softmax(extra["hP"], extra["hL"], s)
        elif name == "softmax_grad_f16":
            G.case_softmax_grad(extra["hG"], extra["hP"], extra["hlab"], s)
        elif name == "sum_rows_f16":    # half_t one is 0x3C00
            G.case_reduce_keep_lowest(extra["h2b"], extra["hM"], 0, 0, 0x3C00, 0, s)
        elif name == "sumall_except_dim1_f16":
            G.case_reduce_keep_highdim(extra["h2a"], extra["hX"], 0, 0, 0x3C00, 0, s)
        elif name == "sumall_except_dim1_64_kept":   # the floats of X2a read as (64,64,112,112)
            G.check(G.dll.mshadow_hip_reduce_keep_highdim_f32(
                cur["out_2a"].ptr, cur["dev"]["X2a"].ptr, 112, 64, 64, 112, 112, 0, 0, 1.0, s))
        elif name == "sumall_except_dim1_16_kept":   # ... and as (256,16,112,112)
            G.check(G.dll.mshadow_hip_reduce_keep_highdim_f32(
                cur["out_2a"].ptr, cur["dev"]["X2a"].ptr, 112, 256, 16, 112, 112, 0, 0, 1.0, s))
        elif name == "dot_f32_4096":
            G.case_dot(1, extra["mm_out"], dev["A"], dev["B"], 4096, 4096, 4096, 1, s)
        elif name == "dot_f16_8192":
            G.blas_gemm(extra["f16"], 1, 0, 8192, 8192, 8192, 1.0, extra["ha"], 8192, extra["hb"], 8192,
                        0.0, extra["hc"], 8192, stream=s)
        elif name == "bias_add_broadcast":
            G.case_shaping(0, extra["out4"], dev["X2a"], extra["bias"], 64, 256, 56, 56, s)
        elif name == "swapaxis10_reshape":
            G.case_shaping(2, extra["out4"], dev["X2a"], extra["bias"], 64, 256, 56, 56, s)
        elif name == "lrn_scale_chpool5":   # x * (chpool<sum>(F<square>(x), 5) * 0.1 + 1)
            G.case_extensions(19, extra["out4"], dev["X2a"], None, None, 64, 256, 56, 56, 5, 0, 0, s)
        elif name == "transpose_nchw_nhwc":
            G.case_extensions(7, extra["out4"], dev["X2a"], None, None, 64, 256, 56, 56, 231, 0, 0, s)
        elif name == "sort_by_key_f32":     # 16M (float key, int value) pairs, ascending
            G.check(G.dll.mshadow_hip_sort_by_key_32(extra["keys"].ptr, 0, extra["vals"].ptr, 1 << 24,
                                                     1, extra["work"].ptr, extra["work_bytes"], s))
        elif name == "smooth_softmax_grad_ignore":
            G.softmax_grad_ex(out_g, out_p, dev["labels"], 3, 17.0, 0.1, s)
        elif name == "softmax3d":
            G.softmax3d(extra["p3"], extra["x3"], s)
        elif name == "softmax3d_grad":
            G.softmax3d_grad(extra["g3"], extra["p3"], extra["l3"], 0, 0.0, 0.0, s)
        elif name == "add_take_grad":
            G.add_take_grad(extra["emb"], extra["idx"], extra["rows"], s)
        elif name == "map_fused":
            G.case_map_fused(cur["out_map"], cur["dev"]["A"], cur["dev"]["B"], cur["dev"]["C"], cur["dev"]["D"], 0, s)
        elif name == "sumall_except_dim1":
            G.reduce_keep_highdim(cur["out_2a"], cur["dev"]["X2a"], stream=s)
        elif name == "sum_rows":
            G.reduce_keep_lowest(cur["out_2b"], cur["dev"]["M2b"], stream=s)
        elif name == "softmax":
            G.softmax(cur["out_p"], cur["dev"]["L"], s)
        elif name == "softmax_grad":
            G.softmax_grad(cur["out_g"], nxt["out_p"], cur["dev"]["labels"], s)
        elif name == "pool_max":
            G.pool(cur["out_pool"], cur["dev"]["X4"], 3, 3, 2, 2, stream=s)
        elif name == "unpool_max":
            G.unpool(cur["out_unpool"], cur["dev"]["X4"], nxt["out_pool"], cur["dev"]["G4"], 3, 3, 2, 2, stream=s)
        elif name == "im2col_f16":
            G.im2col(cur["out_col"], cur["dimg"], 3, 3, 1, 1, 1, 1, 1, 1, s)
        elif name == "col2im_f16":
            G.col2im(cur["out_img"], cur["dcol_in"], 3, 3, 1, 1, 1, 1, 1, 1, s)
        elif name == "calib_copy":
            # one read and one write of 4096x4096 floats: the known-size kernel that the
            # HBM traffic counters are scaled by (only with --only, never part of a step)
            G.case_map_axpb(out_map, dev["A"], 0.0, 1.0, 0.0, 0, s)

    for k in range(args.warmup):
        use_set(k)
        for name in only:
            run_op(name)
    G.stream_sync(s)
    G.device_sync()

    # Per-operation pass (not the timed region): the same K steps with an event after every
    # launch, which gives every operation's interval and names the dominant one. An event
    # between two launches costs the step about 3 us each, so the timed region below keeps
    # only the two around the dominant operation.
    nev = len(only) + 1
    events = [[G.event_create() for _ in range(nev)] for _ in range(args.steps)]
    for k in range(args.steps):
        use_set(k)
        G.event_record(events[k][0], s)
        for i, name in enumerate(only):
            run_op(name)
            G.event_record(events[k][i + 1], s)
    G.stream_sync(s)
    G.device_sync()
    pass_ms = {name: np.array([G.elapsed_ms(events[k][i], events[k][i + 1]) for k in range(args.steps)])
               for i, name in enumerate(only)}
    dominant = max(pass_ms, key=lambda n: pass_ms[n].mean())

    # The timed region: exactly K steps, synchronized on both sides
    dom_events = [(G.event_create(), G.event_create()) for _ in range(args.steps)]
    G.device_sync()
    wall0 = time.perf_counter()
    for k in range(args.steps):
        use_set(k)
        for name in only:
            if name == dominant:
                G.event_record(dom_events[k][0], s)
                run_op(name)
                G.event_record(dom_events[k][1], s)
            else:
                run_op(name)
    G.stream_sync(s)
    G.device_sync()
    wall = time.perf_counter() - wall0
    dom_ms = float(np.mean([G.elapsed_ms(a, b) for a, b in dom_events]))

    # A second figure per operation: the same launch repeated back to back, so that no gap
    # between launches is inside the interval, over three complete sets of operands in turn
    # (3 x 205 MB and more: nothing is found in the 256 MB memory-side cache from the
    # launch before). "ms" above is the operation's interval inside the step, gap included.
    b2b_ms = {}
    if rotate:
        G.stream_sync(s)
        reps = 12
        for name in only:
            ev = [G.event_create(), G.event_create()]
            for r in range(3):
                use_set(r)
                run_op(name)
            G.event_record(ev[0], s)
            for r in range(reps):
                use_set(r)
                run_op(name)
            G.event_record(ev[1], s)
            G.stream_sync(s)
            b2b_ms[name] = G.elapsed_ms(ev[0], ev[1]) / reps
        use_set(0)

    # A third figure for the step: the same launches recorded once into a HIP graph (one step per
    # operand set) and replayed - what a caller that replays a fixed sequence pays per step.
    graph_ms = None
    if rotate and all(o in OPS for o in only):
        try:
            G.graph_begin(s)
            for k in range(len(sets)):
                use_set(k)
                for name in only:
                    run_op(name)
            graph = G.graph_end(s)
            replays = max(1, (args.steps + len(sets) - 1) // len(sets))
            G.graph_launch(graph, s)          # warm-up
            G.stream_sync(s)
            gev = [G.event_create(), G.event_create()]
            G.event_record(gev[0], s)
            for _ in range(replays):
                G.graph_launch(graph, s)
            G.event_record(gev[1], s)
            G.stream_sync(s)
            graph_ms = G.elapsed_ms(gev[0], gev[1]) / (replays * len(sets))
            G.graph_destroy(graph)
        except Exception as e:  # noqa: BLE001 - the figure is an extra; the line must still come out
            print(f"bench.py: graph replay skipped: {e}", file=sys.stderr)
        use_set(0)

    abytes = algorithmic_bytes()
    elems = work_elements()
    scale_fix = 1.0 / args.scale
    per_op = []
    op_ms = {}
    for i, name in enumerate(only):
        ms = pass_ms[name]
        op_ms[name] = float(ms.mean())
        gbs = abytes[name] * scale_fix / (ms.mean() * 1e-3) / 1e9
        per_op.append({"op": name, "ms": round(float(ms.mean()), 4), "ms_min": round(float(ms.min()), 4),
                       "GBps": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
                       "GElemps": round(elems[name] * scale_fix / (ms.mean() * 1e-3) / 1e9, 2)})
        if name in b2b_ms:
            per_op[-1]["ms_back_to_back"] = round(b2b_ms[name], 4)
            per_op[-1]["frac_of_hbm_peak_back_to_back"] = round(
                abytes[name] / (b2b_ms[name] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        if name in ORDER_FAITHFUL:
            per_op[-1].update(ORDER_FAITHFUL[name])
        if name in PRODUCT_FLOPS:
            flops, peak = PRODUCT_FLOPS[name]
            per_op[-1]["TFLOPps"] = round(flops / (ms.mean() * 1e-3) / 1e12, 1)
            per_op[-1]["frac_of_mfma_peak"] = round(per_op[-1]["TFLOPps"] / peak, 4)
    step_ms = wall / args.steps * 1e3
    total_bytes = sum(abytes[n] for n in only) * scale_fix
    value = total_bytes / (step_ms * 1e-3) / 1e9
    dom_gbs = abytes[dominant] * scale_fix / (dom_ms * 1e-3) / 1e9

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(H, img_h, col_h, only, abytes, scale_fix, args.cpu_reps)
        for row in per_op:
            c = cpu["per_op_ms"].get(row["op"])
            if c:
                row["cpu_ms"] = round(c, 2)
                row["speedup_vs_cpu"] = round(c / row["ms"], 1)

    out = {
        "metric": "effective HBM GB/s (algorithmic bytes / time) over the nine hot-path ops",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32 (f16 storage for im2col/col2im)",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs 1-5 at full shape, one pass each per step: "
                               "map 4096x4096 f32; sumall_except_dim<1> (64,256,56,56); sum_rows "
                               "16384x4096; Softmax+SoftmaxGrad 8192x32000; pool/unpool max 3x3 s2 "
                               "(128,64,112,112); im2col/col2im 3x3 s1 p1 (32,256,56,56) f16"
                               + ("" if args.scale == 1 else f" [leading dims / {args.scale}]"),
                   "ops": only, "device": props.name.decode() or props.arch.decode(),
                   "arch": props.arch.decode(), "compute_units": props.compute_units},
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": round(dom_gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(dom_gbs / HBM_PEAK_GBS, 4),
                     "traffic": measured_hbm_bytes(dominant) if args.scale == 1 else None,
                     "traffic_source": os.path.relpath(TRAFFIC_PROFILE, ROOT)},
        "per_op": per_op,
        "input_generation_s": round(gen_s, 1),
    }
    if graph_ms is not None:
        out["ms_per_step_graph_replay"] = round(graph_ms, 4)
    if cpu is not None:
        out["cpu_baseline"] = {k: v for k, v in cpu.items() if k != "per_op_ms"}
    print(json.dumps(out))


def neighbour_shapes(G):
    """`--only neighbour_shapes`: the fixed-function operations on shapes next to the BASELINE
    ones (other windows, strides, paddings, plane sizes, row lengths, float images), each
    launched 10 times on the same buffers after 2 warm-up launches - small operands stay in the
    caches, so these are upper figures. Prints one JSON line: op, shape, us, GB/s over the
    algorithmic bytes, fraction of the HBM peak."""
    s = G.stream_create()
    rng = np.random.default_rng(3)
    rows_out = []

    def timeit(fn, reps=10):
        for _ in range(2):
            fn()
        G.stream_sync(s)
        a, b = G.event_create(), G.event_create()
        G.event_record(a, s)
        for _ in range(reps):
            fn()
        G.event_record(b, s)
        G.event_sync(b)
        return G.elapsed_ms(a, b) / reps * 1e3

    def report(op, shape, nbytes, us):
        rows_out.append({"op": op, "shape": shape, "us": round(us, 1), "GBps": round(nbytes / us / 1e3),
                         "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 3)})

    def big(shape):
        return rng.standard_normal(int(np.prod(shape)), dtype=f32).reshape(shape)

    for shape, k, st in (((128, 64, 112, 112), 2, 2), ((128, 64, 112, 112), 3, 2), ((128, 64, 112, 112), 3, 1),
                         ((64, 96, 55, 55), 3, 2), ((256, 256, 13, 13), 3, 2), ((32, 64, 224, 224), 2, 2),
                         ((128, 256, 28, 28), 2, 2), ((32, 64, 224, 224), 5, 1)):
        n, c, h, w = shape
        ph, pw = (h - k) // st + 1, (w - k) // st + 1
        x = big(shape)
        dx, out = G.to_device(x), G.buffer((n, c, ph, pw), f32)
        report("pool max", f"{shape} k{k} s{st}", x.nbytes + out.nbytes,
               timeit(lambda: G.pool(out, dx, k, k, st, st, stream=s)))
        gr, up = G.to_device(big((n, c, ph, pw))), G.buffer(shape, f32)
        report("unpool max", f"{shape} k{k} s{st}", 2 * x.nbytes + 2 * out.nbytes,
               timeit(lambda: G.unpool(up, dx, out, gr, k, k, st, st, stream=s)))
        del dx, out, gr, up
    for shape, k, st, pad, dt in (((32, 256, 56, 56), 3, 1, 1, f32), ((32, 256, 56, 56), 3, 1, 1, np.uint16),
                                  ((32, 64, 112, 112), 3, 1, 1, np.uint16), ((32, 256, 56, 56), 1, 1, 0, np.uint16),
                                  ((32, 3, 224, 224), 7, 2, 3, f32), ((32, 128, 28, 28), 5, 1, 2, np.uint16),
                                  ((32, 256, 56, 56), 3, 2, 1, np.uint16), ((32, 256, 56, 56), 3, 1, 0, np.uint16)):
        n, c, h, w = shape
        oh, ow = (h + 2 * pad - k) // st + 1, (w + 2 * pad - k) // st + 1
        img = big(shape) if dt == f32 else big(shape).astype(np.float16).view(np.uint16)
        dimg, dcol = G.to_device(img), G.buffer((c * k * k, n * oh * ow), dt)
        tag = f"{shape} k{k} s{st} p{pad} {'f32' if dt == f32 else 'f16'}"
        report("im2col", tag, img.nbytes + dcol.nbytes,
               timeit(lambda: G.im2col(dcol, dimg, k, k, st, st, 1, 1, pad, pad, s)))
        back = G.buffer(shape, dt)
        report("col2im", tag, img.nbytes + dcol.nbytes,
               timeit(lambda: G.col2im(back, dcol, k, k, st, st, 1, 1, pad, pad, s)))
        del dimg, dcol, back
    for shape in ((64, 256, 56, 56), (128, 64, 112, 112), (32, 512, 28, 28), (256, 1000, 1, 1), (64, 2048, 7, 7),
                  (8, 256, 200, 200)):
        x = big(shape)
        dx, out = G.to_device(x), G.buffer((shape[1],), f32)
        report("sumall_except_dim<1>", str(shape), x.nbytes, timeit(lambda: G.reduce_keep_highdim(out, dx, stream=s)))
        del dx, out
    for shape in ((16384, 4096), (256, 1000), (4096, 4096), (65536, 1024), (1024, 65536), (100000, 100), (128, 1 << 20)):
        x = big(shape)
        dx, out = G.to_device(x), G.buffer((shape[1],), f32)
        report("sum_rows", str(shape), x.nbytes, timeit(lambda: G.reduce_keep_lowest(out, dx, stream=s)))
        del dx, out
    for shape in ((8192, 32000), (65536, 1000), (128, 1000), (4096, 4096), (131072, 256), (16384, 2304), (8192, 12288), (2048, 50257), (16, 250000), (512, 128000)):
        x = big(shape) * f32(3)
        dx, out = G.to_device(x), G.buffer(shape, f32)
        report("softmax", str(shape), 2 * x.nbytes, timeit(lambda: G.softmax(out, dx, s)))
        lab, g = G.to_device(rng.integers(0, shape[1], shape[0]).astype(f32)), G.buffer(shape, f32)
        report("softmax_grad", str(shape), 2 * x.nbytes, timeit(lambda: G.softmax_grad(g, out, lab, s)))
        del dx, out, lab, g
    print(json.dumps({"probe": "neighbour_shapes", "unit": "us per launch, 10 launches on the same buffers",
                      "rows": rows_out}))


def run_probe(G, which, pattern=""):
    """`--only softmax_phases`: where a row of the 8192 x 32000 softmax spends its time (time
    stamps taken inside an instrumented build of the library's kernel). `--only ceiling_chain`:
    the cost of one dependent float add for a single wave, alone on the chip and with every CU
    busy - the floor of any kernel that must add in the reference's order, sum_rows first of
    all (16384 dependent adds per column). `--only ceiling_lds_loads`: how fast the loads from
    global memory straight into LDS, which feed the reduction kernels, run with nothing
    consuming the data - per access pattern, bytes per lane and waves per workgroup.
    Prints one JSON line."""
    import mshadow_amd
    P = mshadow_amd.load_probe()
    s = G.stream_create()
    cus = G.props(0).compute_units
    if which == "ceiling_chain":
        out = {"probe": "ceiling_chain", "unit": "ns per dependent float32 add, one wave",
               "compute_units": cus, "modes": {}}
        for mode in ("register", "register_f16", "lds", "lanes"):
            out["modes"][mode] = {f"{wg} workgroups": round(P.add_chain_ns(mode, wg, s), 3)
                                  for wg in (1, cus, 4 * cus)}
        lds = out["modes"]["lds"]
        out["sum_rows_floor_us"] = {k: round(16384 * v * 1e-3, 1) for k, v in lds.items()}
        out["sum_rows_f16_floor_us"] = {k: round(16384 * v * 1e-3, 1)
                                        for k, v in out["modes"]["register_f16"].items()}
    elif which == "ceiling_lds_loads":
        src = G.to_device(np.ones((16384, 4096), f32))
        mb = 16384 * 4096 * 4 / 1e6
        out = {"probe": "ceiling_lds_loads", "matrix": [16384, 4096], "unit": "us to read the matrix once "
               "(GB/s)", "patterns": {}}
        names = {0: "contiguous pieces, 1024 workgroups",
                 -1: "64 segments side by side per workgroup, 256 workgroups"}
        names.update({c: f"{c} columns of every row per workgroup" for c in (16, 32, 64)})
        table = [(strip, width, waves) for strip in (0, -1, 16, 32, 64) for width in (4, 16)
                 for waves in ((4, 8, 16) if width == 4 else (2, 4, 8))]
        if pattern:
            table = [tuple(int(v) for v in pattern.split(":"))]
        for strip, width, waves in table:
            if True:
                if True:
                    us = min(P.dma_rate_us(src, strip, width, waves, s) for _ in range(3))
                    out["patterns"][f"{names[strip]}; {width} bytes per lane; {waves} waves"] = \
                        [round(us, 1), round(mb / us * 1e3)]
    elif which == "ceiling_seg_loads":
        # segments of 3136 floats one after the other as in a (n,c,56,56) tensor; 270 MB, more
        # than the memory-side cache holds, so that a launch finds nothing from the one before
        nseg = 21504
        src = G.to_device(np.ones((nseg, 3136), f32))
        mb = nseg * 3136 * 4 / 1e6
        out = {"probe": "ceiling_seg_loads", "segments": [nseg, 3136],
               "unit": "us to read the segments once (GB/s of what was read)", "patterns": {}}
        for segs in (64, 32, 16, 8):
            for width, waves, piece in ((4, 8, 1), (4, 16, 1), (4, 8, 7), (4, 4, 1), (16, 4, 1), (16, 8, 1),
                                        (16, 8, 4), (16, 4, 4)):
                per_seg = 3136 // (16 * width)
                read = per_seg // piece * piece * 16 * width / 3136.0
                us = min(P.seg_rate_us(src, 3136, nseg, segs, width, waves, piece, s) for _ in range(3))
                out["patterns"][f"{segs} segments per workgroup ({nseg // segs} workgroups); {width} bytes per lane; "
                                f"{waves} waves; pieces of {piece * 64 * width} bytes"] = \
                    [round(us, 1), round(mb * read / us * 1e3)]
    elif which == "highdim_split_configs":
        out = {"probe": "highdim_split_configs", "unit": "us per launch (cold memory-side cache)", "shapes": {}}
        names = {-1: "one workgroup per kept index", 0: "64 segments, 8 loader waves, 8 slots, 4 bytes per lane",
                 1: "32, 8, 8, 4", 2: "16, 8, 4, 16", 3: "32, 8, 4, 16", 4: "16, 4, 8, 4", 5: "32, 8, 6, 4",
                 6: "64, 8, 6, 4", 7: "32, 4, 8, 4", 8: "16, 8, 8, 4"}
        for shape in ((64, 256, 56, 56), (64, 64, 112, 112), (256, 16, 112, 112), (64, 1024, 28, 28)):
            x = np.random.default_rng(5).standard_normal(shape, dtype=f32)
            a, b = G.to_device(x), G.to_device(x)
            dst = G.buffer((shape[1],), f32)
            res = {}
            want = None
            for cfg in sorted(names):
                us = min(P.highdim_split_us(dst, a, b, cfg, s) for _ in range(3))
                got = dst.download(s)
                want = got if want is None else want
                res[names[cfg]] = [round(us, 1), bool(np.array_equal(got.view(np.uint32), want.view(np.uint32)))]
            out["shapes"]["x".join(map(str, shape))] = res
    elif which == "staying_waves_copy":
        # 1 GiB copied by waves that stay until it is done: each wave on a contiguous run of its own
        # (as many sequential streams as waves) against the waves side by side on one moving region
        floats = 1 << 28
        src, dst = G.buffer((8192, 32768), f32), G.buffer((8192, 32768), f32)
        G.fill(src, 1.0, s)
        out = {"probe": "staying_waves_copy", "bytes_read": floats * 4, "bytes_written": floats * 4,
               "unit": "us per copy; fraction of the HBM peak", "variants": {}}
        for per_cu in (1, 2, 4, 8):
            wgs = per_cu * cus
            for own_run, name in ((1, "own contiguous run per wave"), (0, "waves side by side")):
                us = min(P.stream_copy_us(dst, src, floats, wgs, own_run, s) for _ in range(3))
                out["variants"][f"{wgs} workgroups of 4 waves, {name}"] = [
                    round(us, 1), round(2 * floats * 4 / us / 1e3 / HBM_PEAK_GBS, 3)]
        # and by 65536 workgroups that move 16 KB each and end
        out["short_lived_workgroups_us"] = round(min(P.stream_copy_us(dst, src, floats, floats // (4 * 256 * 4), 1, s)
                                                     for _ in range(3)), 1)
    elif which == "softmax_prefetch_copy":
        L = np.random.default_rng(7).standard_normal((8192, 32000), dtype=f32) * f32(3)
        src, dst = G.to_device(L), G.buffer(L.shape, f32)
        out = {"probe": "softmax_prefetch_copy", "shape": [8192, 32000], "unit": "us per copy of the matrix",
               "row_copy_two_rows_per_cu": round(min(P.row_copy_us(dst, src, 0, 0, s) for _ in range(3)), 1),
               "variants": {}}
        for threads, pre, wgs in ((1024, 8, cus), (1024, 4, cus), (512, 8, 2 * cus), (512, 4, 2 * cus),
                                  (512, 16, cus), (512, 4, 3 * cus)):
            for barriers, spin in ((0, 0), (4, 4), (8, 8), (8, 16)):
                us = min(P.row_copy_prefetch_us(dst, src, threads, pre, barriers, spin, wgs, s) for _ in range(3))
                out["variants"][f"{threads} threads, {pre} KB per wave ahead in LDS, {wgs} workgroups; "
                                f"{barriers} barriers x {spin} multiply-adds"] = round(us, 1)
        G.fill(dst, 0.0, s)
        P.row_copy_prefetch_us(dst, src, 1024, 8, 2, 0, cus, s)
        ok = np.array_equal(dst.download(s), L)
        G.fill(dst, 0.0, s)
        P.row_copy_prefetch_us(dst, src, 512, 8, 2, 0, 2 * cus, s)
        out["copy_is_exact"] = bool(ok and np.array_equal(dst.download(s), L))
    else:
        L = np.random.default_rng(7).standard_normal((8192, 32000), dtype=f32) * f32(3)
        src, dst = G.to_device(L), G.buffer(L.shape, f32)
        steps, resident, kernel, fallback = P.softmax_phases(dst, src, s)
        G.softmax(dst, src, s)   # the library's own kernel beside it, by HIP events
        ev = [G.event_create() for _ in range(2)]
        G.event_record(ev[0], s)
        for _ in range(10):
            G.softmax(dst, src, s)
        G.event_record(ev[1], s)
        G.stream_sync(s)
        out = {"probe": "softmax_phases", "shape": [8192, 32000],
               "unit": "us, mean over rows, since the previous step (thread 0 of the row)",
               "steps": {k: round(v, 2) for k, v in steps.items()},
               "row_resident_us": round(resident, 2), "instrumented_kernel_us": round(kernel, 1),
               "library_kernel_us": round(G.elapsed_ms(ev[0], ev[1]) * 100.0, 1),
               "rows_in_flight": 2 * cus, "fallback_rows": fallback,
               # the kernel's loads and stores alone, and with stand-in work between them
               "row_copy_us": {f"{b} barriers x {k} multiply-adds per element":
                               round(P.row_copy_us(dst, src, b, k, s), 1)
                               for b, k in ((0, 0), (4, 0), (4, 2), (4, 4), (4, 8), (8, 4))},
               "row_copy_one_row_per_cu_us": round(min(P.row_copy_us(dst, src, 0, 0, s, 1) for _ in range(3)), 1)}
        # how long the steps take when a row has its CU to itself, on 8 and on 16 waves
        # ... and with three rows per CU on four waves each (128 floats of the row per thread)
        for variant, name in ((1, "one_row_per_cu_512_threads"), (2, "one_row_per_cu_1024_threads"),
                              (3, "three_rows_per_cu_256_threads")):
            st, res, ker, fb = P.softmax_phases(dst, src, s, variant)
            out[name] = {"steps": {k: round(v, 2) for k, v in st.items()}, "row_resident_us": round(res, 2),
                         "kernel_us": round(ker, 1), "fallback_rows": fb}
    print(json.dumps(out))


def cpu_baseline(H, img_h, col_h, only, abytes, scale_fix, reps):
    """The same nine operations on the host: the reference's own headers where the
    reference-built library is present ("reference"), the C restatement otherwise
    ("port"). One warm-up pass, then `reps` timed passes over the full inputs. The only part
    of this script that loads anything from oracle/."""
    from checkers import Checker, have_ref
    kind = "reference" if have_ref() else "port"
    cpu = Checker("ref" if kind == "reference" else "orc")
    o_map = np.empty_like(H["A"])
    o_2a, o_2b = np.empty(256, f32), np.empty(4096, f32)
    o_p, o_g = np.empty_like(H["L"]), np.empty_like(H["L"])
    o_pool, o_un = np.empty_like(H["G4"]), np.empty_like(H["X4"])
    o_col, o_img = np.empty_like(col_h), np.empty_like(img_h)
    fns = {
        "map_fused": lambda: cpu.map_fused(o_map, H["A"], H["B"], H["C"], H["D"]),
        "sumall_except_dim1": lambda: cpu.reduce_keep_highdim(o_2a, H["X2a"]),
        "sum_rows": lambda: cpu.reduce_keep_lowest(o_2b, H["M2b"]),
        "softmax": lambda: cpu.softmax(o_p, H["L"]),
        "softmax_grad": lambda: cpu.softmax_grad(o_g, o_p, H["labels"]),
        "pool_max": lambda: cpu.pool(o_pool, H["X4"], 3, 3, 2, 2),
        "unpool_max": lambda: cpu.unpool(o_un, H["X4"], o_pool, H["G4"], 3, 3, 2, 2),
        "im2col_f16": lambda: cpu.im2col(o_col, img_h, 3, 3, 1, 1, 1, 1, 1, 1),
        "col2im_f16": lambda: cpu.col2im(o_img, col_h, 3, 3, 1, 1, 1, 1, 1, 1),
    }
    cpu.softmax(o_p, H["L"])
    cpu.pool(o_pool, H["X4"], 3, 3, 2, 2)
    per = {}
    only = [n for n in only if n in fns]
    for name in only:
        fns[name]()  # warm-up
        t = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fns[name]()
            t.append(time.perf_counter() - t0)
        per[name] = float(np.mean(t)) * 1e3
    total_ms = sum(per.values())
    total_bytes = sum(abytes[n] for n in only) * scale_fix
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": round(total_bytes / (total_ms * 1e-3) / 1e9, 2), "unit": "GB/s",
            "cores": cpu.num_threads(), "kind": kind,
            "sample": f"all ops of the step at full shape, mean of {reps} passes after 1 warm-up "
                      f"({total_ms:.0f} ms per pass)",
            "cpu_model": model, "per_op_ms": per}


if __name__ == "__main__":
    main()
