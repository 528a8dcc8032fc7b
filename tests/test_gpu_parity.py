"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle.

Every test feeds the same seeded arrays to the oracle (oracle/liboracle.so, and the
reference-built library where it is present) and to the GPU. Two GPU routes are checked:
the fixed-function entry points of libmshadow_hip.so (include/mshadow_hip.h) and the C++
expression API (Tensor<gpu> expressions compiled in libmshadow_cases.so), the latter both
on the recognised fast path (variant 0) and through the generic expression kernel
(variant 1).

Bars: bit-exact for the elementwise map, pool / unpool, patch2col / col2patch, the
softmax gradient and - because the kernels keep the CPU path's order of additions - the
reductions. Softmax forward is compared at relative 1e-5 (the tolerance of the task);
its only source of difference is expf (libm on the host, the device math library here).
"""
import numpy as np
import pytest

from checkers import DIVTO, MAX, MIN, MINUSTO, MULTO, PLUSTO, SAVETO, SUM, Checker, have_ref
from gpu_util import assert_bits_equal, f32, host_padded, normal, uniform

pytestmark = pytest.mark.gpu


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


@pytest.fixture(scope="module")
def O():
    return Checker("orc")


def test_device_is_gfx950(G):
    p = G.props(0)
    assert b"gfx950" in p.arch, p.arch
    assert p.wavefront_size == 64
    print("device:", p.name.decode(), p.arch.decode(), "CUs", p.compute_units, "LDS/block",
          p.lds_bytes_per_block)


def test_reference_library_agrees_with_oracle_on_this_host(O):
    """The reference-built checker travels as a binary; make sure it still matches here."""
    if not have_ref():
        pytest.skip("oracle/_ref not present")
    R = Checker("ref")
    a, b, c, d = (uniform(100 + i, (64, 257)) for i in range(4))
    o1, o2 = np.empty_like(a), np.empty_like(a)
    O.map_fused(o1, a, b, c, d)
    R.map_fused(o2, a, b, c, d)
    assert_bits_equal(o1, o2, "ref vs oracle map")
    x = normal(104, (16, 4000), 3.0)
    s1, s2 = np.empty_like(x), np.empty_like(x)
    O.softmax(s1, x)
    R.softmax(s2, x)
    assert_bits_equal(s1, s2, "ref vs oracle softmax")


# ------------------------------------------------------------------ copy / alloc
@pytest.mark.parametrize("shape,pad", [((7, 55), 0), ((7, 55), 1), ((33, 64), 1), ((3, 1000), 1),
                                       ((1, 5), 1)])
def test_copy_roundtrip_and_pitch(G, shape, pad):
    a = uniform(1, shape)
    out, stride = G.case_copy_roundtrip(a, pad)
    assert_bits_equal(out, a, "copy round trip")
    if pad and shape[1] >= 64:
        assert stride % 64 == 0 and stride >= shape[1]  # 256-byte pitch
    else:
        assert stride == shape[1]


@pytest.mark.parametrize("rows,width,dpitch,spitch,doff,soff", [
    (7, 220, 220, 224, 0, 0),          # 4-byte units, different pitches
    (33, 256, 512, 272, 0, 0),         # whole 16-byte packs, pitched on both sides
    (21, 1000, 1016, 1008, 8, 0),      # 8-byte units
    (5, 4000, 4000, 4000, 0, 0),       # dense: one run
    (1, 4004, 4004, 4004, 0, 0),       # a single row keeps its width, whatever the pitch says
    (3, 1001, 1008, 1003, 0, 0),       # an odd number of bytes: the runtime's copy
    (9, 64, 96, 80, 2, 6),             # addresses that are no multiple of 4: the runtime's copy
    (700, 128000, 128000, 128256, 0, 0),
    (650, 127960, 128000, 128000, 0, 0)])
def test_device_to_device_copy_of_pitched_views(G, stream, rows, width, dpitch, spitch, doff, soff):
    """mshadow_hip_memcpy2d_async device to device: exactly the bytes of the view arrive, the
    gaps between rows and around the view keep their contents"""
    from mshadow_amd.capi import D2D
    rng = np.random.default_rng(rows * 31 + width)
    src_host = rng.integers(0, 256, rows * spitch + 64, dtype=np.uint8)
    dst_host = rng.integers(0, 256, rows * dpitch + 64, dtype=np.uint8)
    src, dst = G.to_device(src_host), G.to_device(dst_host)
    G.check(G.dll.mshadow_hip_memcpy2d_async(dst.ptr + doff, dpitch, src.ptr + soff, spitch, width, rows,
                                             D2D, stream))
    want = dst_host.copy()
    for y in range(rows):
        want[doff + y * dpitch: doff + y * dpitch + width] = src_host[soff + y * spitch: soff + y * spitch + width]
    assert np.array_equal(dst.download(stream), want)


def test_copy_between_device_tensors_through_the_header_api(G, stream):
    """Copy(Tensor<gpu>, Tensor<gpu>, stream) with either side pitched"""
    a = uniform(3, (37, 300))
    for spad, dpad in ((0, 0), (4, 0), (0, 12), (5, 3)):
        src = G.to_device(a, spad)
        dst = G.to_device(np.zeros_like(a), dpad)
        G.case_copy_d2d(dst, src, stream)
        assert_bits_equal(dst.download(stream), a, f"Copy pads {spad} {dpad}")


# ------------------------------------------------------------------ elementwise map
MAP_SHAPES = [((4096 // 8, 4096 // 8), 0), ((257, 515), 0), ((257, 516), 4), ((33, 7), 1),
              ((1, 1), 0), ((5, 1024), 0), ((129, 260), 12)]


@pytest.mark.parametrize("shape,pad", MAP_SHAPES)
@pytest.mark.parametrize("saver", [SAVETO, PLUSTO, MINUSTO, MULTO, DIVTO])
def test_map_fused(G, O, stream, shape, pad, saver):
    a, b, c, d = (uniform(10 + i, shape) for i in range(4))
    start = np.random.default_rng(14).uniform(1, 2, shape).astype(f32)
    want = host_padded(start, pad)
    O.map_fused(want, host_padded(a, pad), host_padded(b, pad), host_padded(c, pad),
                host_padded(d, pad), saver)
    da, db, dc, dd = (G.to_device(t, pad) for t in (a, b, c, d))
    dst = G.to_device(start, pad)
    G.case_map_fused(dst, da, db, dc, dd, saver, stream)
    assert_bits_equal(dst.download(stream), want, f"map {shape} pad {pad} saver {saver}")


def test_map_mixed_strides_and_misaligned_pointer(G, O, stream):
    """Leaves with different pitches (pack kernel, row-indexed) and an odd column count
    (scalar kernel)."""
    for shape, pads in (((64, 256), (0, 4, 8, 12, 16)), ((64, 255), (0, 1, 2, 3, 0))):
        a, b, c, d = (uniform(20 + i, shape) for i in range(4))
        want = np.empty(shape, f32)
        O.map_fused(want, a, b, c, d)
        bufs = [G.to_device(t, p) for t, p in zip((a, b, c, d), pads[:4])]
        dst = G.buffer(shape, f32, pads[4])
        G.case_map_fused(dst, *bufs, SAVETO, stream)
        assert_bits_equal(dst.download(stream), want, f"mixed strides {shape}")


@pytest.mark.parametrize("saver", [SAVETO, PLUSTO, MULTO, DIVTO])
def test_map_scalar_and_axpb(G, O, stream, saver):
    shape = (37, 300)
    start = uniform(30, shape) + f32(2)
    a = uniform(31, shape)
    want = start.copy()
    O.map_scalar(want, 1.7, saver)
    dst = G.to_device(start, 4)
    G.case_map_scalar(dst, 1.7, saver, stream)
    assert_bits_equal(dst.download(stream), want, "scalar rhs")
    want = start.copy()
    O.map_axpb(want, a, 10.0, 3.0, 2.0, saver)
    dst = G.to_device(start, 0)
    G.case_map_axpb(dst, G.to_device(a), 10.0, 3.0, 2.0, saver, stream)
    assert_bits_equal(dst.download(stream), want, "axpb")


def test_map_shape_mismatch_is_an_error(G, stream):
    from mshadow_amd import HipError
    a = G.to_device(uniform(1, (4, 8)))
    dst = G.buffer((4, 8), f32)
    # lie about the shape of dst through the raw entry: rows differ between dst and sources
    import ctypes as C
    st = G.cases.mshadow_case_softmax_f32(dst.ptr, 8, a.ptr, 8, 4, 8, stream)
    assert st == 0
    with pytest.raises(HipError):
        G.check(G.dll.mshadow_hip_softmax_f32(dst.ptr, 4, a.ptr, 8, 4, 8, stream))  # pitch < cols


# ------------------------------------------------------------------ reductions
LOWEST_SHAPES = [((16384 // 8, 4096 // 8), 0), ((1000, 37), 3), ((1, 130), 0), ((257, 16), 0),
                 ((255, 1), 1), ((4097, 48), 0), ((2500, 19), 2)]


@pytest.mark.parametrize("shape,pad", LOWEST_SHAPES)
@pytest.mark.parametrize("reducer", [SUM, MAX, MIN])
@pytest.mark.parametrize("route", ["abi", "expr", "expr_generic"])
def test_reduce_keep_lowest(G, O, stream, shape, pad, reducer, route):
    m = normal(40, shape)
    for saver, scale in ((SAVETO, 1.0), (PLUSTO, 0.75)):
        start = uniform(41, (shape[1],)) + f32(2)
        want = start.copy()
        O.reduce_keep_lowest(want, host_padded(m, pad), reducer, saver, scale)
        dst = G.to_device(start)
        src = G.to_device(m, pad)
        if route == "abi":
            G.reduce_keep_lowest(dst, src, reducer, saver, scale, stream)
        else:
            G.case_reduce_keep_lowest(dst, src, reducer, saver, scale,
                                      1 if route == "expr_generic" else 0, stream)
        assert_bits_equal(dst.download(stream), want, f"keep_lowest {shape} {route}")


HIGH_SHAPES = [((8, 32, 56, 56), 0), ((64, 5, 7, 9), 2), ((3, 4, 5, 6), 0), ((1, 3, 2, 4), 0),
               ((70, 3, 1, 1), 0), ((17, 2, 33, 65), 3), ((2, 2, 70, 70), 0),
               # long enough for the direct-to-LDS kernels, one shape per segment count
               ((70, 3, 33, 65), 3), ((5, 2, 130, 129), 0), ((2, 2, 200, 200), 0),
               ((1, 2, 300, 300), 1),
               # rows of whole 16-byte packs: the inner chains are dealt out in groups of 16
               # segments (dense; pitched; more groups than kept indices; a last group that is
               # not full; segments of one pack; more inner results than the scratch memory holds)
               ((64, 7, 32, 36), 0), ((33, 5, 40, 52), 4), ((300, 1, 16, 16), 0),
               ((20000, 3, 1, 4), 0), ((70000, 1, 1, 4), 0), ((9, 40, 90, 100), 0),
               # a kept index for every CU: one workgroup each, no merge
               ((40, 200, 41, 40), 0)]


@pytest.mark.parametrize("shape,pad", HIGH_SHAPES)
@pytest.mark.parametrize("reducer", [SUM, MAX, MIN])
@pytest.mark.parametrize("route", ["abi", "expr", "expr_generic"])
def test_reduce_keep_highdim(G, O, stream, shape, pad, reducer, route):
    x = normal(50, shape)
    for saver, scale in ((SAVETO, 1.0), (MINUSTO, 1.25)):
        start = uniform(51, (shape[1],)) + f32(2)
        want = start.copy()
        O.reduce_keep_highdim(want, host_padded(x, pad), reducer, saver, scale)
        dst = G.to_device(start)
        src = G.to_device(x, pad)
        if route == "abi":
            G.reduce_keep_highdim(dst, src, reducer, saver, scale, stream)
        else:
            G.case_reduce_keep_highdim(dst, src, reducer, saver, scale,
                                       1 if route == "expr_generic" else 0, stream)
        assert_bits_equal(dst.download(stream), want, f"keep_highdim {shape} {route}")


def test_reduce_keep_highdim_on_more_streams_than_scratch_slots(G, O):
    """every stream gets the same result, whether it was given scratch memory for the inner
    results (the first eight of a GPU) or runs the kernel that needs none; a slot is free again
    once its stream is destroyed"""
    shape = (40, 6, 48, 64)
    x = normal(52, shape)
    want = np.empty(shape[1], f32)
    O.reduce_keep_highdim(want, x, SUM, SAVETO, 1.0)
    src = G.to_device(x)
    for _ in range(2):
        streams = [G.stream_create() for _ in range(11)]
        outs = [G.buffer((shape[1],), f32) for _ in streams]
        for st, dst in zip(streams, outs):
            G.reduce_keep_highdim(dst, src, SUM, SAVETO, 1.0, st)
            G.reduce_keep_highdim(dst, src, SUM, SAVETO, 1.0, st)   # the counter is zero again
        for st, dst in zip(streams, outs):
            assert_bits_equal(dst.download(st), want, "keep_highdim, many streams")
            G.stream_destroy(st)


def test_reduce_reference_known_answers(G, stream):
    # test/test.cu:9-18,35,47 of the reference
    i, j, k = np.meshgrid(np.arange(3), np.arange(2), np.arange(4), indexing="ij")
    tc = (f32(0.1) * i.astype(f32) + f32(0.2) * j.astype(f32) + f32(0.1) * k.astype(f32))
    out = G.buffer((4,), f32)
    G.case_reduce_keep_lowest(out, G.to_device(tc[0]), SUM, SAVETO, 1.0, 0, stream)
    assert np.allclose(out.download(stream), [0.2, 0.4, 0.6, 0.8], atol=1e-4)
    out3 = G.buffer((3,), f32)
    G.case_reduce_keep_highdim(out3, G.to_device(tc.reshape(1, 3, 2, 4)), SUM, SAVETO, 1.0, 0,
                               stream)
    assert np.allclose(out3.download(stream), [2.0, 2.8, 3.6], atol=1e-4)


# ------------------------------------------------------------------ softmax
SOFTMAX_SHAPES = [((64, 32000), 0), ((5, 1000), 0), ((5, 1001), 0), ((3, 7), 1), ((9, 2048), 4),
                  ((4, 8192), 0), ((3, 16384), 0), ((2, 40000), 0), ((2, 70001), 0), ((7, 1), 0),
                  ((3, 5000), 3), ((2, 20000), 1),
                  # rows that neither start at multiples of 16 bytes nor are whole packs
                  ((3, 50257), 0), ((2, 33333), 1), ((2, 65535), 0), ((6, 4097), 2), ((5, 1023), 0),
                  # rows longer than a workgroup's registers hold: stretch by stretch (two, four and five stretches,
                  # a last stretch of one column, of one pack, pitched rows)
                  ((3, 128000), 0), ((2, 200001), 1), ((1, 262149), 0), ((2, 65537), 3), ((2, 65540), 0), ((2, 131072), 2),
                  # many rows of a few hundred to 2048 columns: a wave per row, slab after slab
                  ((2100, 300), 0), ((2049, 777), 3), ((2050, 1024), 0), ((2048, 2047), 1), ((4100, 513), 0),
                  # ... up to 3072 columns; many rows of 8193 to 16384 columns: four waves a row
                  ((2100, 2304), 0), ((2050, 3072), 1), ((2049, 2999), 0), ((4100, 8200), 0), ((4096, 12001), 0),
                  # short rows: one thread per row up to 32 columns, one wave per row up to 256
                  ((1000, 10), 0), ((300, 32), 0), ((77, 33), 2), ((130, 64), 0), ((50, 65), 1),
                  ((41, 128), 0), ((19, 200), 3), ((64, 256), 0), ((9, 257), 0), ((5, 2), 0),
                  # ... four rows to a wave (33 to 128 columns) and two (129 to 256), thousands of them, pitched rows,
                  # row counts that leave the last wave partly empty
                  ((5003, 100), 1), ((3001, 250), 0), ((4099, 48), 3), ((2050, 129), 2), ((1, 256), 0), ((3, 40), 0)]


def _softmax_check(got, want, src):
    rel = np.abs(got.astype(np.float64) - want) / np.maximum(want, np.finfo(f32).tiny)
    mask = want > 0
    assert np.all(got[~mask] == 0) or np.allclose(got[~mask], want[~mask], atol=1e-44)
    worst = rel[mask].max() if mask.any() else 0.0
    assert worst <= 1e-5, f"softmax relative error {worst:.3e} > 1e-5 (tolerance of the task)"
    return worst


@pytest.mark.parametrize("shape,pad", SOFTMAX_SHAPES)
def test_softmax_forward(G, O, stream, shape, pad):
    x = normal(60, shape, 3.0)
    want = np.empty(shape, f32)
    O.softmax(want, x)
    src = G.to_device(x, pad)
    dst = G.buffer(shape, f32, pad)
    G.softmax(dst, src, stream)
    got = dst.download(stream)
    worst = _softmax_check(got, want, x)
    # through Softmax(Tensor<gpu,2>, Tensor<gpu,2>) and in place
    G.case_softmax(src, src, stream)
    assert_bits_equal(src.download(stream), got, "in-place softmax via the C++ API")
    print(f"softmax {shape} pad {pad}: worst relative difference to the CPU path {worst:.2e}")


def test_softmax_exact_cases(G, stream):
    # uniform logits: exp(0) = 1 exactly, the sum of n ones is exact, so every output is 1/n
    for n in (4, 7, 1000, 32000):
        x = np.full((3, n), 0.37, f32)
        dst = G.buffer(x.shape, f32)
        G.softmax(dst, G.to_device(x), stream)
        assert np.all(dst.download(stream) == f32(1.0) / f32(n))
    # a row of distinct powers of two in exp-space is too contrived; instead: the row sum
    # the kernel used must be the left-to-right float sum of ITS OWN exponentials.
    x = normal(61, (8, 32000), 3.0)
    dst = G.buffer(x.shape, f32)
    G.softmax(dst, G.to_device(x), stream)
    got = dst.download(stream)
    for y in range(8):
        k = int(np.argmax(x[y]))
        s = f32(1.0) / got[y, k]          # exp(0) / sum
        # reconstruct p_i = got_i * s only approximately; the check is on the order effect:
        p = np.exp((x[y] - x[y].max()).astype(np.float64))
        exact = p.sum()
        seq_bias = (float(s) - exact) / exact
        # the sequential float sum sits ~2.6e-5 below the exact sum on this distribution;
        # a tree sum would sit within 1e-6 of it
        assert -6e-5 < seq_bias < -5e-6, seq_bias


def _serial_row_sums(O, terms):
    """strictly left-to-right float32 sums of each row (the oracle's keep-dimension fold)"""
    rows, cols = terms.shape
    want = np.empty(rows, f32)
    O.reduce_keep_highdim(want, np.ascontiguousarray(terms).reshape(1, rows, 1, cols), SUM, SAVETO, 1.0)
    return want


ROWSUM_COLS = [1, 3, 10, 31, 32, 33, 64, 65, 128, 129, 255, 256, 257, 300, 513, 777, 1000, 1024, 1028, 2048, 2049, 2304, 3000,
               3072, 3073, 4096, 5001, 8192, 8196, 12000, 16384,
               20001, 32000, 32768, 40000, 65536,
               # longer than a workgroup's registers hold: summed stretch by stretch, each from the sum in front
               65537, 70001, 131072, 131075, 200001, 262149]


@pytest.mark.parametrize("cols", ROWSUM_COLS)
def test_softmax_rowsum_is_the_serial_sum(G, O, stream, cols):
    """the row-sum stage of Softmax, fed with terms directly, against a serial float sum:
    bit for bit, on terms shaped like a softmax's and on ones built to hit ties, long runs
    of zeros, many binade crossings in one chunk and sums that end next to a power of two"""
    rng = np.random.default_rng(1000 + cols)
    rows = []
    for sigma in (0.1, 1.0, 3.0, 10.0, 40.0):
        x = rng.standard_normal(cols) * sigma
        rows.append(np.exp(x - x.max()))
    rows.append(rng.uniform(0, 1, cols))
    rows.append(np.full(cols, 1.0))                               # exact integers
    rows.append(np.ldexp(rng.integers(1, 9, cols).astype(np.float64), -3))   # multiples of 1/8: ties
    rows.append(np.ldexp(rng.integers(0, 3, cols).astype(np.float64), -24) + (np.arange(cols) == 0))
    z = rng.uniform(0, 1, cols)
    z[: cols // 2] = 0.0                                          # leading zeros
    rows.append(z)
    rows.append(np.ldexp(1.0, rng.integers(-40, 20, cols)))       # huge dynamic range
    rows.append(np.where(np.arange(cols) % 97 == 0, 1.0, 1e-7))   # rare large terms
    rows.append(np.zeros(cols))
    t = np.zeros(cols)
    t[-1] = 3.5
    rows.append(t)
    rows.append(np.full(cols, 2.0 ** -130))                       # subnormal terms
    terms = np.asarray(rows, dtype=f32)
    want = _serial_row_sums(O, terms)
    for pad in (0, 1):
        sums = G.buffer((terms.shape[0],), f32)
        G.softmax_rowsum(sums, G.to_device(terms, pad), stream)
        assert_bits_equal(sums.download(stream), want, f"row sum cols={cols} pad={pad}")
    if 256 < cols <= 3072:
        # with thousands of rows these lengths take the kernel with a wave per row
        many = np.tile(terms, (150, 1))
        sums = G.buffer((many.shape[0],), f32)
        G.softmax_rowsum(sums, G.to_device(many, 1), stream)
        assert_bits_equal(sums.download(stream), np.tile(want, 150), f"row sum cols={cols}, a wave per row")
    if 8192 < cols <= 16384 and cols % 4 == 0:
        # and these, as whole packs, the workgroup of four waves with 64 columns a thread
        many = np.tile(terms, (260, 1))
        sums = G.buffer((many.shape[0],), f32)
        G.softmax_rowsum(sums, G.to_device(many), stream)
        assert_bits_equal(sums.download(stream), np.tile(want, 260), f"row sum cols={cols}, four waves a row")


def test_softmax_rowsum_specials(G, O, stream):
    cols = 5000
    base = np.random.default_rng(7).uniform(0, 1, cols).astype(f32)
    rows = []
    for pos in (0, 17, 2500, cols - 1):
        for val in (np.inf, np.nan, -0.5, 3.0e38):
            r = base.copy()
            r[pos] = val
            rows.append(r)
    terms = np.asarray(rows, dtype=f32)
    want = _serial_row_sums(O, terms)
    sums = G.buffer((terms.shape[0],), f32)
    G.softmax_rowsum(sums, G.to_device(terms), stream)
    got = sums.download(stream)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all(), (got, want)


def test_softmax_rowsum_specials_in_long_rows(G, O, stream):
    """rows summed stretch by stretch: a negative, infinite, huge or NaN term in any stretch gives what
    the serial loop gives (the plan is for non-negative terms; anything else is summed by wave scans,
    from the sum of the stretches in front)"""
    cols = 100003
    base = np.random.default_rng(8).uniform(0, 1, cols).astype(f32)
    rows = []
    for pos in (3, 32767, 32768, 70000, cols - 1):
        for val in (np.inf, np.nan, -0.5, 3.0e38):
            r = base.copy()
            r[pos] = val
            rows.append(r)
    terms = np.asarray(rows, dtype=f32)
    want = _serial_row_sums(O, terms)
    sums = G.buffer((terms.shape[0],), f32)
    G.softmax_rowsum(sums, G.to_device(terms), stream)
    got = sums.download(stream)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all(), (got, want)


def test_softmax_extreme_rows(G, O, stream):
    rows = [
        np.linspace(-200, 0, 5000),          # long underflowing head (leading zeros)
        np.linspace(0, -200, 5000),
        np.concatenate([np.full(10, -1e30), [0.0], np.full(300, -90.0)]),  # denormal terms
        np.full(777, -3.0e38),               # all equal, huge magnitude
        np.r_[np.zeros(4000), 50.0],         # sum dominated by the last term
    ]
    for r in rows:
        x = np.asarray(r, dtype=f32)[None, :]
        want = np.empty_like(x)
        O.softmax(want, x)
        dst = G.buffer(x.shape, f32)
        G.softmax(dst, G.to_device(x), stream)
        got = dst.download(stream)
        big = want > 1e-30
        rel = np.abs(got[big].astype(np.float64) - want[big]) / want[big]
        assert rel.max() <= 1e-5
        assert np.all(np.abs(got[~big].astype(np.float64) - want[~big]) <= 1e-35)


def test_softmax_long_rows_extremes_and_specials(G, O, stream):
    """rows taken stretch by stretch: the maximum in the last stretch, a long underflowing head, one
    class far above the rest in a middle stretch; a NaN or an infinite logit makes the row NaN as on
    the CPU, wherever it sits"""
    n = 150000
    rng = np.random.default_rng(77)
    base = (rng.standard_normal(n) * 3).astype(f32)
    rows = [np.linspace(-300, 0, n), np.linspace(0, -300, n), np.r_[np.full(n - 1, -5.0), 40.0], base.copy(), base.copy()]
    rows[3][70000] = 60.0
    rows[4][140000] = 25.0
    x = np.asarray(rows, dtype=f32)
    want = np.empty_like(x)
    O.softmax(want, x)
    dst = G.buffer(x.shape, f32)
    G.softmax(dst, G.to_device(x), stream)
    got = dst.download(stream)
    rel = np.abs(got.astype(np.float64) - want) / np.maximum(want, np.finfo(f32).tiny)
    assert rel.max() <= 1e-5, rel.max()
    for pos in (5, 40000, 100000, n - 1):
        for val in (np.nan, np.inf):
            y = base.copy()[None, :]
            y[0, pos] = val
            O.softmax(want[:1], y)
            G.softmax(dst, G.to_device(np.repeat(y, 5, 0)), stream)
            got = dst.download(stream)
            assert np.isnan(want[0]).all() and np.isnan(got).all(), (pos, val)
    y = base.copy()[None, :]
    y[0, 90000] = -np.inf            # a class that cannot occur: its probability is 0, the rest as usual
    O.softmax(want[:1], y)
    G.softmax(dst, G.to_device(np.repeat(y, 5, 0)), stream)
    got = dst.download(stream)
    assert got[2, 90000] == 0.0 and want[0, 90000] == 0.0
    rel = np.abs(got[2].astype(np.float64) - want[0]) / np.maximum(want[0], np.finfo(f32).tiny)
    assert rel.max() <= 1e-5


@pytest.mark.parametrize("shape,pad", [((64, 32000), 0), ((9, 1001), 0), ((9, 1000), 4),
                                       ((5, 7), 1), ((3, 20000), 0)])
def test_softmax_grad(G, O, stream, shape, pad):
    rng = np.random.default_rng(62)
    p = rng.uniform(0, 1, shape).astype(f32)
    label = rng.integers(0, shape[1], shape[0]).astype(f32)
    if shape[0] > 4:
        label[1], label[2], label[3] = shape[1] + 5, -3.0, 0.9
    want = np.empty(shape, f32)
    O.softmax_grad(want, p, label)
    for route in ("abi", "expr"):
        dst = G.buffer(shape, f32, pad)
        args = (dst, G.to_device(p, pad), G.to_device(label))
        (G.softmax_grad if route == "abi" else G.case_softmax_grad)(*args, stream)
        assert_bits_equal(dst.download(stream), want, f"softmax_grad {shape} {route}")


# ------------------------------------------------------------------ pool / unpool
POOL_CASES = [  # planes, h, w, ky, kx, sy, sx, pad
    (16, 112, 112, 3, 3, 2, 2, 0), (6, 37, 41, 3, 3, 2, 2, 2), (6, 37, 41, 2, 2, 2, 2, 0),
    (3, 9, 11, 3, 2, 1, 3, 1), (2, 30, 30, 5, 5, 3, 2, 0), (4, 6, 6, 1, 1, 1, 1, 0),
    (2, 7, 300, 7, 3, 1, 2, 0), (1, 3, 20000, 2, 2, 1, 2, 0),
    # many small planes: several per workgroup, the last workgroup with fewer
    (4096, 9, 9, 3, 3, 2, 2, 0), (2560, 13, 13, 3, 3, 2, 2, 1), (2500, 7, 10, 2, 2, 2, 2, 0),
    (3001, 12, 70, 3, 2, 1, 2, 2),
    # 2 x 2 stride 2 on even and odd sizes, narrow and wide rows
    (5, 40, 44, 2, 2, 2, 2, 3), (7, 41, 43, 2, 2, 2, 2, 0), (3, 9, 6, 2, 2, 2, 2, 1), (2, 8, 5, 2, 2, 2, 2, 0),
    (2, 6, 258, 2, 2, 2, 2, 0),
    # 3 x 3 stride 2 on odd heights, rows that are not whole packs, pitches, one to 64 packs per row
    (96, 55, 55, 3, 3, 2, 2, 0), (40, 27, 27, 3, 3, 2, 2, 3), (5, 8, 5, 3, 3, 2, 2, 0), (3, 7, 256, 3, 3, 2, 2, 0),
    (3, 6, 254, 3, 3, 2, 2, 1), (70, 3, 3, 3, 3, 2, 2, 0), (9, 14, 18, 3, 3, 2, 2, 2), (4, 5, 260, 3, 3, 2, 2, 0),
    # stride 1, 3 x 3 and 2 x 2. Planes of 64 to 256 pixels a side: strips of rows (16 to 64 packs per row, planes
    # that end inside a strip, rows that end inside a pack, pitches); smaller and wider ones: the staged kernels
    (16, 112, 112, 3, 3, 1, 1, 0), (6, 70, 67, 3, 3, 1, 1, 2), (3, 65, 256, 3, 3, 1, 1, 0), (4, 80, 130, 2, 2, 1, 1, 0),
    (2, 64, 64, 2, 2, 1, 1, 3), (700, 64, 66, 3, 3, 1, 1, 1), (5, 97, 201, 3, 3, 1, 1, 0),
    (6, 37, 41, 3, 3, 1, 1, 2), (5, 20, 256, 3, 3, 1, 1, 0), (7, 9, 4, 3, 3, 1, 1, 0), (3, 5, 7, 2, 2, 1, 1, 1),
    (2560, 13, 13, 3, 3, 1, 1, 0), (3, 66, 260, 3, 3, 1, 1, 0), (300, 28, 28, 3, 3, 1, 1, 3),
    # stride 1 in the pooling kernels that walk down output columns: rows of whole packs (four columns a thread,
    # dense and pitched by a multiple of four) and others, 5 x 5, bands that end early, fewer than 16 outputs a row
    (4, 64, 112, 5, 5, 1, 1, 0), (3, 40, 130, 5, 5, 1, 1, 1), (2, 131, 64, 3, 3, 1, 1, 4), (5, 57, 57, 3, 3, 1, 1, 0),
    (3, 50, 20, 5, 5, 1, 1, 0), (2, 300, 16, 2, 2, 1, 1, 0), (2, 47, 1024, 3, 3, 1, 1, 0), (3, 33, 68, 2, 2, 1, 1, 8),
]


@pytest.mark.parametrize("case", POOL_CASES)
@pytest.mark.parametrize("reducer", [MAX, MIN, SUM])
@pytest.mark.parametrize("variant", [0, 1])
def test_pool_unpool(G, O, stream, case, reducer, variant):
    planes, h, w, ky, kx, sy, sx, pad = case
    if variant == 1 and w > 1000:
        pytest.skip("generic route covered by the smaller shapes")
    rng = np.random.default_rng(70 + h + w)
    # a coarse value grid makes duplicated maxima common, which equality routing must honour
    src = (rng.integers(-8, 9, (planes, h, w)).astype(f32) / f32(8)) if h < 100 else \
        uniform(71, (planes, h, w))
    ph, pw = (h - ky) // sy + 1, (w - kx) // sx + 1
    want = np.empty((planes, ph, pw), f32)
    O.pool(want, host_padded(src, pad), ky, kx, sy, sx, reducer)
    dsrc = G.to_device(src, pad)
    dpool = G.buffer((planes, ph, pw), f32, pad)
    G.case_pool(dpool, dsrc, ky, kx, sy, sx, reducer, variant, stream)
    assert_bits_equal(dpool.download(stream), want, f"pool {case}")
    grad = normal(72, (planes, ph, pw))
    wantu = np.empty((planes, h, w), f32)
    O.unpool(wantu, src, want, grad, ky, kx, sy, sx, reducer)
    dgrad = G.to_device(grad, pad)
    dun = G.buffer((planes, h, w), f32, pad)
    G.case_unpool(dun, dsrc, dpool, dgrad, ky, kx, sy, sx, reducer, variant, stream)
    assert_bits_equal(dun.download(stream), wantu, f"unpool {case}")
    if variant == 0:  # and straight through the C ABI
        d2 = G.buffer((planes, ph, pw), f32)
        G.pool(d2, dsrc, ky, kx, sy, sx, reducer, stream)
        assert_bits_equal(d2.download(stream), want, "pool abi")
        u2 = G.buffer((planes, h, w), f32)
        G.unpool(u2, dsrc, dpool, dgrad, ky, kx, sy, sx, reducer, stream)
        assert_bits_equal(u2.download(stream), wantu, "unpool abi")


@pytest.mark.parametrize("case", [(4100, 56, 60, 3), (2100, 64, 64, 2), (2300, 41, 100, 5)])
@pytest.mark.parametrize("reducer", [MAX, MIN, SUM])
def test_pool_stride1_many_planes_zero_signs(G, O, stream, case, reducer):
    """stride-1 pooling over thousands of dense planes of one band each; some planes hold zeros of both
    signs, where max and min go by the reference's comparison, the others do not"""
    planes, h, w, k = case
    rng = np.random.default_rng(planes + k)
    src = rng.integers(-5, 6, (planes, h, w)).astype(f32) / f32(4)
    some = src[::7]
    some[rng.random(some.shape) < 0.05] = f32(-0.0)
    src[::7] = some
    ph, pw = h - k + 1, w - k + 1
    want = np.empty((planes, ph, pw), f32)
    O.pool(want, src, k, k, 1, 1, reducer)
    dpool = G.buffer((planes, ph, pw), f32)
    G.pool(dpool, G.to_device(src), k, k, 1, 1, reducer, stream)
    assert_bits_equal(dpool.download(stream), want, f"pool {case}")


@pytest.mark.parametrize("case", [(40, 70, 66, 3, 2), (40, 70, 66, 3, 1), (30, 65, 130, 2, 1), (30, 64, 64, 5, 1),
                                  (900, 13, 13, 3, 2), (900, 13, 13, 3, 1), (24, 50, 52, 2, 2), (6, 40, 45, 4, 3)])
@pytest.mark.parametrize("reducer", [MAX, MIN, SUM])
def test_pool_special_values(G, O, stream, case, reducer):
    """NaN, infinities, the largest finite values and subnormals as window members in every staged pool
    kernel, in planes with zeros of both signs (max and min by the reference's comparison) and in planes
    with none (by single instructions): both pass over a NaN and agree bit for bit"""
    planes, h, w, k, st = case
    rng = np.random.default_rng(planes + 10 * k + st)
    src = rng.integers(-3, 4, (planes, h, w)).astype(f32) / f32(2)
    src[src == 0] = f32(0.25)
    specials = np.array([np.nan, np.inf, -np.inf, 3.4028235e38, -3.4028235e38, 1e-45, -1e-45], f32)
    where = rng.random(src.shape) < 0.3
    src[where] = specials[rng.integers(0, specials.size, int(where.sum()))]
    src[0, :4, :] = np.nan      # windows of NaN only
    zeros = src[1::2]           # every second plane: zeros of both signs too
    zw = rng.random(zeros.shape) < 0.2
    zeros[zw] = np.where(rng.random(int(zw.sum())) < 0.5, f32(-0.0), f32(0.0))
    src[1::2] = zeros
    ph, pw = (h - k) // st + 1, (w - k) // st + 1
    want = np.empty((planes, ph, pw), f32)
    O.pool(want, src, k, k, st, st, reducer)
    dpool = G.buffer((planes, ph, pw), f32)
    G.pool(dpool, G.to_device(src), k, k, st, st, reducer, stream)
    got = dpool.download(stream)
    if reducer == SUM:  # a NaN sum is a NaN on both sides; its sign and payload are the adder's own
        assert np.array_equal(np.isnan(got), np.isnan(want)), f"pool {case}: NaN in other places"
        got, want = np.where(np.isnan(got), f32(0), got), np.where(np.isnan(want), f32(0), want)
    else:
        assert not np.isnan(want).any()
    assert_bits_equal(got, want, f"pool {case}")


@pytest.mark.parametrize("shape", [(3, 9, 12, 3, 4), (3, 9, 12, 4, 5), (2, 10, 16, 2, 7), (2, 11, 13, 5, 3),
                                   (4, 8, 8, 3, 3), (5, 6, 10, 2, 4), (2, 70, 72, 60, 66), (3, 64, 100, 31, 97)])
@pytest.mark.parametrize("reducer", [MAX, SUM])
def test_unpool_given_pooled_shape(G, O, stream, shape, reducer):
    """unpool with a pooled grid the caller names (smaller than the natural one): only its windows count"""
    planes, h, w, ph, pw = shape
    for ky, kx, sy, sx in ((3, 3, 2, 2), (2, 2, 2, 2), (3, 3, 1, 1), (2, 2, 1, 1)):
        if (ph - 1) * sy + ky > h or (pw - 1) * sx + kx > w:
            continue
        rng = np.random.default_rng(500 + h * w + ph)
        src = rng.integers(-8, 9, (planes, h, w)).astype(f32) / f32(8)
        pooled = np.empty((planes, ph, pw), f32)
        O.pool(pooled, src, ky, kx, sy, sx, reducer)
        grad = normal(73, (planes, ph, pw))
        want = np.empty((planes, h, w), f32)
        O.unpool(want, src, pooled, grad, ky, kx, sy, sx, reducer)
        out = G.buffer((planes, h, w), f32)
        G.unpool(out, G.to_device(src), G.to_device(pooled), G.to_device(grad), ky, kx, sy, sx, reducer, stream)
        assert_bits_equal(out.download(stream), want, f"unpool {shape} k{ky} s{sy}")


def test_pool_reference_known_answers(G, stream):
    # test/pool.cu:29-48 of the reference: 6x6 0.1i+0.1j, 2x2 stride 2 -> src[2a+1][2b+1]
    i, j = np.meshgrid(np.arange(6), np.arange(6), indexing="ij")
    src = (i.astype(f32) * f32(0.1) + j.astype(f32) * f32(0.1)).reshape(1, 6, 6)
    out = G.buffer((1, 3, 3), f32)
    G.case_pool(out, G.to_device(src), 2, 2, 2, 2, MAX, 0, stream)
    assert np.array_equal(out.download(stream)[0], src[0, 1::2, 1::2])
    # explicit pooled shape larger than natural: windows past the edge keep -FLT_MAX
    out = G.buffer((1, 4, 4), f32)
    G.pool(out, G.to_device(src), 2, 2, 2, 2, MAX, stream)
    got = out.download(stream)
    assert np.array_equal(got[0, :3, :3], src[0, 1::2, 1::2])
    assert np.all(got[0, 3, :] == -np.finfo(f32).max) and np.all(got[0, :, 3] == -np.finfo(f32).max)


# ------------------------------------------------------------------ im2col / col2im
CONV = [  # n, c, h, w, ky, kx, sy, sx, dy, dx, py, px
    (2, 16, 56, 56, 3, 3, 1, 1, 1, 1, 1, 1), (3, 5, 19, 23, 3, 3, 2, 2, 1, 1, 0, 0),
    (3, 5, 19, 23, 5, 3, 2, 1, 1, 1, 2, 1), (2, 3, 19, 23, 3, 3, 1, 1, 2, 2, 2, 2),
    (2, 3, 9, 8, 2, 3, 1, 2, 2, 2, 1, 0), (1, 1, 6, 6, 3, 3, 2, 2, 1, 1, 0, 0),
    (2, 4, 7, 7, 1, 1, 1, 1, 1, 1, 0, 0), (1, 2, 30, 31, 7, 7, 3, 3, 1, 1, 3, 3),
    # dense rows of whole packs, staged pack by pack: many small planes; 5 taps down; planes
    # cut into several bands of rows
    (40, 64, 16, 16, 3, 3, 1, 1, 1, 1, 1, 1), (3, 700, 8, 24, 5, 3, 1, 1, 1, 1, 2, 1),
    (1, 2, 300, 128, 3, 3, 1, 1, 1, 1, 1, 1), (2, 1, 181, 264, 4, 3, 1, 1, 1, 1, 2, 1),
    # stride 1 with patch rows that are not whole packs, no padding, wide windows, odd sizes
    (2, 5, 54, 54, 3, 3, 1, 1, 1, 1, 0, 0), (3, 4, 28, 28, 5, 5, 1, 1, 1, 1, 2, 2),
    (8, 3, 13, 17, 3, 5, 1, 1, 1, 1, 0, 2), (8, 2, 9, 9, 7, 7, 1, 1, 1, 1, 3, 3),
    (16, 6, 10, 12, 1, 1, 1, 1, 1, 1, 0, 0), (8, 2, 6, 40, 2, 4, 1, 1, 1, 1, 1, 3),
    # strides and dilations on rows of a pack or more
    (4, 6, 56, 56, 3, 3, 2, 2, 1, 1, 1, 1), (2, 3, 64, 70, 7, 7, 2, 2, 1, 1, 3, 3),
    (3, 2, 40, 44, 3, 3, 1, 1, 2, 2, 2, 2), (2, 2, 45, 50, 3, 5, 3, 2, 2, 1, 1, 2),
    # a step of two between patches in a row: dilated taps, rows of odd length, no padding, padding wider than a pack
    (2, 3, 50, 61, 3, 3, 1, 2, 1, 2, 1, 2), (3, 2, 33, 35, 1, 1, 2, 2, 1, 1, 0, 0), (2, 2, 30, 47, 5, 5, 2, 2, 1, 1, 0, 9),
    (2, 3, 33, 47, 11, 11, 4, 4, 1, 1, 0, 0),
    # col2im with a step of two along x, the patches of every second pixel from one 8-byte load: windows of even
    # and odd width from 3 to 8, rows of odd length (the last pack moved back starts at an odd pixel), the patch
    # grid as narrow as one load, other steps along y, padding wider than the window; 9 wide: the general kernel.
    # Steps of 3: every load issued before the first add, 1 to 4 patches over a pixel in each direction
    (2, 3, 40, 64, 7, 7, 2, 2, 1, 1, 3, 3), (2, 2, 31, 45, 4, 4, 2, 2, 1, 1, 1, 1), (3, 2, 20, 37, 8, 8, 2, 2, 1, 1, 4, 4),
    (2, 2, 19, 11, 3, 3, 2, 2, 1, 1, 0, 0), (2, 2, 16, 8, 3, 3, 2, 2, 1, 1, 0, 0), (2, 3, 33, 52, 5, 5, 3, 2, 1, 1, 2, 2),
    (2, 2, 26, 38, 3, 6, 1, 2, 1, 1, 1, 7), (1, 2, 30, 41, 9, 9, 2, 2, 1, 1, 4, 4), (2, 2, 28, 28, 2, 2, 2, 2, 1, 1, 0, 0),
    (2, 3, 34, 40, 3, 3, 3, 3, 1, 1, 1, 1), (2, 2, 35, 43, 7, 5, 3, 3, 1, 1, 3, 2), (1, 2, 40, 48, 11, 11, 3, 3, 1, 1, 5, 5),
    # im2col with all taps of a tap row from one fetch (3, 5, 7 taps with a step of two; 5, 7 with a step of one):
    # dilated tap rows, steps between rows, padding wider than a pack, odd widths, the patch row as short as one pack
    (2, 3, 30, 33, 3, 5, 2, 1, 2, 1, 2, 2), (2, 2, 24, 40, 5, 7, 1, 1, 1, 1, 0, 3), (1, 3, 21, 29, 2, 7, 3, 2, 1, 1, 1, 9),
    (2, 2, 17, 19, 3, 5, 1, 2, 1, 1, 0, 0), (2, 2, 12, 12, 5, 5, 1, 1, 1, 1, 0, 0), (2, 2, 18, 21, 1, 3, 2, 2, 1, 1, 0, 10),
    (2, 3, 32, 32, 4, 4, 2, 2, 1, 1, 1, 1), (3, 2, 21, 35, 4, 4, 2, 2, 1, 1, 0, 2),
]


@pytest.mark.parametrize("cfg", CONV)
@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("variant", [0, 1])
def test_im2col_col2im(G, O, stream, cfg, dtype, variant):
    n, c, h, w, ky, kx, sy, sx, dy, dx, py, px = cfg
    shape = Checker.col_shape(n, c, h, w, ky, kx, sy, sx, dy, dx, py, px)
    imgf = uniform(80, (n, c, h, w))
    colf = normal(81, shape)
    if dtype == "f16":
        img, colin, dt = O.float2half(imgf), O.float2half(colf), np.uint16
    else:
        img, colin, dt = imgf, colf, f32
    for pad in (0, 3):
        want = np.empty(shape, dt)
        O.im2col(want, img, ky, kx, sy, sx, dy, dx, py, px)
        dcol = G.buffer(shape, dt, pad)
        G.case_im2col(dcol, G.to_device(img, pad), ky, kx, sy, sx, dy, dx, py, px, variant, stream)
        assert_bits_equal(dcol.download(stream), want, f"im2col {cfg} {dtype} pad {pad}")
        wanti = np.empty((n, c, h, w), dt)
        O.col2im(wanti, colin, ky, kx, sy, sx, dy, dx, py, px)
        dimg = G.buffer((n, c, h, w), dt, pad)
        G.case_col2im(dimg, G.to_device(colin, pad), ky, kx, sy, sx, dy, dx, py, px, variant,
                      stream)
        assert_bits_equal(dimg.download(stream), wanti, f"col2im {cfg} {dtype} pad {pad}")
    if variant == 0:
        dcol = G.buffer(shape, dt)
        G.im2col(dcol, G.to_device(img), ky, kx, sy, sx, dy, dx, py, px, stream)
        assert_bits_equal(dcol.download(stream), want, "im2col abi")
        dimg = G.buffer((n, c, h, w), dt)
        G.col2im(dimg, G.to_device(colin), ky, kx, sy, sx, dy, dx, py, px, stream)
        assert_bits_equal(dimg.download(stream), wanti, "col2im abi")


def test_im2col_reference_known_answer(G, stream):
    # test/unpack.cu:29-59 of the reference
    i, j = np.meshgrid(np.arange(6), np.arange(6), indexing="ij")
    img = (i.astype(f32) * f32(0.1) + j.astype(f32) * f32(0.2)).reshape(1, 1, 6, 6)
    col = G.buffer((9, 4), f32)
    G.case_im2col(col, G.to_device(img), 3, 3, 2, 2, 1, 1, 0, 0, 0, stream)
    got = col.download(stream)
    for ky in range(3):
        for kx in range(3):
            for oy in range(2):
                for ox in range(2):
                    assert got[ky * 3 + kx, oy * 2 + ox] == img[0, 0, 2 * oy + ky, 2 * ox + kx]


@pytest.mark.gpu
def test_fill_of_more_than_2_to_the_31_elements(G, stream):
    """`tensor = scalar` on 8.6 GB: the entry point launches runs of whole rows; the first and
    last rows, the rows on either side of a run boundary and a guard row behind the tensor
    are read back"""
    rows, cols = (1 << 15) + 3, (1 << 16) + 1      # odd rows: one element per store, 32767 rows per run
    buf = G.buffer((rows + 1, cols), np.float32)
    G.fill(buf, 0.0, stream)            # the whole allocation, guard row included
    bits = int(np.array([2.5], np.float32).view(np.uint32)[0])
    G.check(G.dll.mshadow_hip_fill_32(buf.ptr, cols, rows, cols, bits, stream))
    per_run = ((1 << 31) - 1) // cols
    assert 1 < per_run < rows
    from mshadow_amd.capi import D2H
    for r, want in ((0, 2.5), (1, 2.5), (per_run - 1, 2.5), (per_run, 2.5), (rows - 1, 2.5), (rows, 0.0)):
        out = np.empty(cols, np.float32)
        G.check(G.dll.mshadow_hip_memcpy2d_async(out.ctypes.data, cols * 4, buf.ptr + r * cols * 4, cols * 4,
                                                 cols * 4, 1, D2H, stream))
        G.stream_sync(stream)
        assert np.all(out == np.float32(want)), r
    buf.free()
