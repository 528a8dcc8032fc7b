"""chpool / ch_unpool, reduce_with_axis / reduce_keepdim, broadcast_with_axis / broadcast_keepdim,
transpose / transpose_indices, concat / slice / flip (as values and as assignment targets),
take / take_grad / one_hot_encode / mat_choose_row_element / mat_fill_row_element / mask / range:
the expressions of mshadow_case_extensions_f32 against plain numpy index loops, on the
reference build (CPU, where present) and on the GPU through the generic expression kernel.
Every result is data movement or a short fixed-order float32 chain: bit for bit."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

from checkers import have_ref

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
f32 = np.float32
SHAPES = [(2, 6, 3, 5), (3, 5, 2, 8), (1, 7, 1, 4)]
BIG = (8, 16, 14, 28)
# rows of whole 128-bit packs with channel counts around the 8 planes a thread of the
# plane-walking kernel takes, and an odd height: the pack-evaluating paths of every node
PACKED = [(2, 12, 5, 12), (4, 9, 7, 16), (1, 33, 2, 4), (3, 8, 4, 20)]


# ---- numpy statements of what each node means (mshadow/extension/*.h of the reference)
def _chpool(a, nsize, stride, pad, reducer):
    n, ch, h, w = a.shape
    pc = (ch - nsize + 2 * pad + 1) // stride
    init = f32(0) if reducer == "sum" else f32(-np.finfo(f32).max)
    out = np.full((n, pc, h, w), init, f32)
    for c in range(pc):
        first = max(c * stride - pad, 0)
        last = min(c * stride - pad + nsize, pc, ch)   # cut at the pooled channel count
        for cc in range(first, last):
            out[:, c] = out[:, c] + a[:, cc] if reducer == "sum" else np.maximum(out[:, c], a[:, cc])
    return out


def _ch_unpool(a, pooled, grad, nsize, stride, pad, reducer):
    n, ch, h, w = a.shape
    out = np.zeros_like(a)
    for c in range(ch):
        reach = nsize - pad
        first = 0 if c < reach else (c - reach + stride) // stride
        # cut at the source channel count (the reference stops there and can run past the
        # pooled tensor; this backend also stops at the pooled channel count)
        last = min((c + pad + stride) // stride, ch, pooled.shape[1])
        for cc in range(first, last):
            pg = np.ones_like(a[:, c]) if reducer == "sum" else (a[:, c] == pooled[:, cc]).astype(f32)
            out[:, c] = out[:, c] + pg * grad[:, cc]
    return out


def _seq_reduce(a, axis, reducer):
    moved = np.moveaxis(a, axis, 0)
    if reducer == "sum":
        res = np.zeros(moved.shape[1:], f32)
        for k in range(moved.shape[0]):
            res = res + moved[k]
        return res
    return moved.min(axis=0) if reducer == "min" else moved.max(axis=0)


def _perm(p0):
    return (p0 // 1000, p0 // 100 % 10, p0 // 10 % 10, p0 % 10)


class Case(object):
    """inputs, parameters and the expected output of one op on one shape"""

    def __init__(self, op, shape):
        n, ch, h, w = shape
        rng = np.random.default_rng(1000 * op + sum(shape))
        a = rng.standard_normal(shape).astype(f32)
        self.op, self.shape, self.a = op, shape, a
        self.b = self.c = None
        self.p = (0, 0, 0)
        self.pitch_pad = 0   # ops 28..31: rows of `a` and of the result are this much apart more
        rows = n * ch * h
        if op == 0:
            self.p = (3, 0, 0)
            self.want = _chpool(a, 3, 1, 1, "sum")
        elif op == 1:
            self.p = (3, 2, 1)
            self.want = _chpool(a, 3, 2, 1, "max")
        elif op in (2, 3):
            # window 5, pad 2 keeps the channel count (the only kind of window for which the
            # reference stays inside the pooled tensor); the large shape, checked on the GPU
            # only, uses a strided window
            self.p = (3, 2, 1) if shape == BIG else (5, 1, 2)
            red = "sum" if op == 2 else "max"
            self.b = _chpool(a, *self.p, red)
            self.c = rng.standard_normal(self.b.shape).astype(f32)
            self.want = _ch_unpool(a, self.b, self.c, *self.p, red)
        elif op == 4:
            self.p = (1 + sum(shape) % 3, 0, 0)
            self.want = _seq_reduce(a, self.p[0], "sum")
        elif op == 5:
            self.p = (sum(shape) % 4, 0, 0)
            self.want = a.argmax(axis=self.p[0]).astype(f32)
        elif op == 6:
            self.p = ((sum(shape) + 1) % 4, 0, 0)
            self.want = np.expand_dims(_seq_reduce(a, self.p[0], "min"), self.p[0])
        elif op == 7:
            self.p = ([2031, 3102, 1230][sum(shape) % 3], 0, 0)
            self.want = a.transpose(_perm(self.p[0]))
        elif op == 8:
            k = ch // 2
            self.p = (k, 0, 0)
            two = a * f32(2)
            self.want = np.concatenate([two[:, :k].ravel(), two[:, k:].ravel()])
        elif op == 9:
            self.p = (2, 0, 0)
            self.b = rng.standard_normal((n, 2, h, w)).astype(f32)
            self.want = np.concatenate([a, self.b], axis=1) + f32(1)
        elif op == 10:
            self.p = (1, ch - 1, 0)
            self.want = a[:, 1:ch - 1]
        elif op == 11:
            self.p = (1, ch - 1, 0)
            self.b = rng.standard_normal(shape).astype(f32)
            self.c = rng.standard_normal((n, ch - 2, h, w)).astype(f32)
            self.want = self.b.copy()
            self.want[:, 1:ch - 1] = self.c * f32(3)
        elif op == 12:
            self.p = (3, 0, 0)
            self.b = rng.standard_normal((n, ch, h, 3)).astype(f32)
            self.want = np.concatenate([a, self.b], axis=3)
        elif op == 13:
            self.p = (1, w - 1, 0)
            self.want = a[..., 1:w - 1]
        elif op == 14:
            self.p = (2, h - 1, 1)
            self.want = a[:, 2:, h - 1:, 1:]
        elif op == 15:
            self.p = (sum(shape) % 4, 0, 0)
            self.want = np.flip(a + f32(0.5), axis=self.p[0])
        elif op == 16:
            self.p = ((sum(shape) + 2) % 4, 0, 0)
            self.want = np.flip(a, axis=self.p[0])
        elif op == 17:
            axis = sum(shape) % 4 - 1
            self.p = (axis, 3, 0)
            a3 = a.reshape(n * ch, h, w)
            self.want = np.repeat(np.expand_dims(a3, axis + 1), 3, axis=axis + 1)
        elif op == 18:
            axis = sum(shape) % 4
            self.p = (axis, 3, 0)
            self.b = np.ascontiguousarray(np.take(a, [0], axis=axis))
            self.want = np.repeat(self.b, 3, axis=axis)
        elif op == 19:
            self.p = (3, 0, 0)
            self.want = a * (_chpool(a * a, 3, 1, 1, "sum") * f32(0.1) + f32(1))
        elif op == 20:
            k = 7
            self.p = (k, 0, 0)
            self.b = rng.integers(0, rows, k).astype(f32)
            self.want = a.reshape(rows, w)[self.b.astype(int)]
        elif op == 21:
            k, dim = min(rows, 9), 4
            self.p = (k, dim, 0)
            self.b = rng.integers(0, dim, k).astype(f32)
            src = a.reshape(rows, w)[:k]
            self.want = np.zeros((dim, w), f32)
            for i in range(k):
                self.want[int(self.b[i])] = self.want[int(self.b[i])] + src[i]
        elif op == 22:
            k, choices = 6, 5
            self.p = (k, choices, 0)
            self.b = rng.integers(0, choices, k).astype(f32)
            self.want = (np.arange(choices)[None, :] == self.b.astype(int)[:, None]).astype(f32)
        elif op == 23:
            self.b = rng.integers(0, w, rows).astype(f32)
            self.want = a.reshape(rows, w)[np.arange(rows), self.b.astype(int)]
        elif op == 24:
            self.b = rng.integers(0, w, rows).astype(f32)
            self.c = rng.standard_normal(rows).astype(f32)
            self.want = a.reshape(rows, w).copy()
            self.want[np.arange(rows), self.b.astype(int)] = self.c
        elif op == 25:
            self.b = rng.integers(0, 2, rows).astype(f32)
            self.want = a.reshape(rows, w) * self.b[:, None]
        elif op == 26:
            self.p = (2, 2 + sum(shape), 3)
            count = -(-(self.p[1] - self.p[0]) // self.p[2])
            self.want = np.repeat(f32(self.p[0]) + np.arange(count).astype(f32) * f32(self.p[2]), 2)
        elif op == 44:
            # four running sums over the multiple-of-4 prefix, folded (s0 + s2) + (s1 + s3), then
            # the tail one by one
            k = h * w
            self.b = rng.standard_normal((k, w)).astype(f32)
            lhs, rhs = a.reshape(n * ch, k), self.b * f32(0.5)
            part = np.zeros((4, n * ch, w), f32)
            whole = k // 4 * 4
            for i in range(whole):
                part[i % 4] = part[i % 4] + lhs[:, i:i + 1] * rhs[i:i + 1, :]
            res = (part[0] + part[2]) + (part[1] + part[3])
            for i in range(whole, k):
                res = res + lhs[:, i:i + 1] * rhs[i:i + 1, :]
            self.want = res
        elif op >= 32:
            # complex numbers as (real, imaginary) pairs along the last dimension
            if w % 2:
                pytest.skip("complex operands need an even last dimension")
            a2 = a.reshape(rows, w)
            self.b = rng.standard_normal((rows, w)).astype(f32)
            self.c = rng.standard_normal((rows, w // 2)).astype(f32)
            ar, ai, br, bi, cr = a2[:, 0::2], a2[:, 1::2], self.b[:, 0::2], self.b[:, 1::2], self.c
            zero = np.zeros_like(cr)

            def pairs(re, im):
                out = np.empty((rows, 2 * re.shape[1]), f32)
                out[:, 0::2], out[:, 1::2] = re, im
                return out

            def mul(xr, xi, yr, yi):
                return pairs(xr * yr - xi * yi, xr * yi + yr * xi)

            def div(xr, xi, yr, yi):
                den = yr * yr + yi * yi
                return pairs((xr * yr + xi * yi) / den, (yr * xi - xr * yi) / den)

            self.want = {
                32: lambda: mul(ar, ai, br, bi), 33: lambda: mul(ar, ai, cr, zero),
                34: lambda: mul(cr, zero, ar, ai), 35: lambda: div(ar, ai, br, bi),
                36: lambda: div(ar, ai, cr, zero), 37: lambda: div(cr, zero, ar, ai),
                38: lambda: pairs(ar, -ai), 39: lambda: pairs(ai, ar),
                40: lambda: pairs(a2, np.zeros_like(a2)), 41: lambda: ar,
                42: lambda: ar * ar + ai * ai, 43: lambda: ar + ai,
            }[op]()
        elif op >= 28:
            # a pitch that keeps 16-byte alignment (pack route where the row length allows it)
            # or one that breaks it (element-wise route)
            self.pitch_pad = 4 if sum(shape) % 2 else 1
            if op == 28:
                self.p = (0, 0, self.pitch_pad)
                self.b = rng.standard_normal(ch).astype(f32)
                self.want = a + self.b.reshape(1, ch, 1, 1)
            elif op == 29:
                self.p = (3, 0, self.pitch_pad)
                self.want = _chpool(a, 3, 1, 1, "sum")
            elif op == 30:
                self.p = (1, ch - 1, self.pitch_pad)
                self.want = a[:, 1:ch - 1]
            else:
                self.p = (0, 0, self.pitch_pad)
                self.want = a.transpose(0, 2, 1, 3)
        else:
            k = 11
            perm = [2031, 3102, 1230][sum(shape) % 3]
            self.p = (perm, k, 0)
            flat = rng.integers(0, a.size, k)
            self.b = flat.astype(f32)
            pos = np.unravel_index(flat, shape)
            axes = _perm(perm)
            tshape = tuple(shape[x] for x in axes)
            self.want = np.ravel_multi_index(tuple(pos[x] for x in axes), tshape).astype(f32)
        self.want = np.ascontiguousarray(self.want, dtype=f32)


N_OPS = 45


def _pitched(arr, pad):
    """the array laid out with `pad` unused elements behind every row (NaN there)"""
    rows = arr.reshape(-1, arr.shape[-1])
    out = np.full((rows.shape[0], rows.shape[1] + pad), np.nan, f32)
    out[:, :rows.shape[1]] = rows
    return out


def _run_on_host(call, case):
    """runs `call(out, a)` on host arrays, through pitched copies for the pitched ops"""
    if not case.pitch_pad:
        out = np.full(case.want.shape, np.nan, f32)
        call(out, case.a)
        return out
    out = _pitched(np.full(case.want.shape, np.nan, f32), case.pitch_pad)
    call(out, _pitched(case.a, case.pitch_pad))
    return np.ascontiguousarray(out[:, :case.want.shape[-1]]).reshape(case.want.shape)


@pytest.fixture(scope="module")
def host_lib(tmp_path_factory):
    """the same expressions on Tensor<cpu> of this backend's headers, compiled with g++"""
    so = str(tmp_path_factory.mktemp("hostcases") / "libhostcases.so")
    cmd = ["g++", "-std=c++17", "-O2", "-fopenmp", "-ffp-contract=off", "-mf16c", "-fPIC", "-shared",
           "-DDMLC_LOG_FATAL_THROW=1", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "mshadow_amd"), "-o", so,
           os.path.join(ROOT, "tests", "host", "ext_cpu_cases.cc")]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    lib = ctypes.CDLL(so)
    fp = ctypes.c_void_p
    lib.host_extensions_f32.argtypes = [ctypes.c_int, fp, fp, fp, fp] + [ctypes.c_int] * 7
    return lib


def _ptr(x):
    return x.ctypes.data_as(ctypes.c_void_p) if x is not None else None


@pytest.mark.parametrize("shape", SHAPES + [BIG] + PACKED)
@pytest.mark.parametrize("op", range(N_OPS))
def test_cpu_device_matches_numpy(host_lib, shape, op):
    case = Case(op, shape)

    def call(out, a):
        assert host_lib.host_extensions_f32(op, _ptr(out), _ptr(a), _ptr(case.b), _ptr(case.c),
                                            *shape, *case.p) == 0
    out = _run_on_host(call, case)
    assert np.array_equal(out.view(np.uint32), case.want.view(np.uint32)), (op, shape)


@pytest.mark.skipif(not have_ref(), reason="reference build absent")
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("op", [o for o in range(N_OPS) if o != 15])
def test_reference_build_matches_numpy(ref, shape, op):
    case = Case(op, shape)
    out = _run_on_host(lambda o, a: ref.extensions(op, o, a, case.b, case.c, *shape, *case.p), case)
    assert np.array_equal(out.view(np.uint32), case.want.view(np.uint32)), (op, shape)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", SHAPES + [BIG] + PACKED)
@pytest.mark.parametrize("op", range(N_OPS))
def test_gpu_matches_numpy(shape, op):
    import mshadow_amd
    G = mshadow_amd.load_cases()
    G.set_device(0)
    case = Case(op, shape)
    out = G.to_device(np.full(case.want.shape, np.nan, f32), pad=case.pitch_pad)
    dev = lambda x: G.to_device(x) if x is not None else None
    G.case_extensions(op, out, G.to_device(case.a, pad=case.pitch_pad), dev(case.b), dev(case.c),
                      *shape, *case.p)
    got = out.download()
    assert np.array_equal(got.view(np.uint32), case.want.view(np.uint32)), (op, shape)


# channel windows where a thread of the plane-walking kernel evaluates 8 adjacent planes at once:
# channel counts above, at and below 8, not multiples of 8 (a group of planes that crosses into
# the next image, a short last group), windows of 3 and 5 (fetches shared in registers) and 7
WINDOW_SHAPES = [(3, 20, 4, 8), (2, 16, 5, 12), (1, 9, 2, 4), (2, 8, 3, 4), (5, 3, 2, 4), (1, 64, 7, 28),
                 (2, 24, 1, 4), (3, 11, 3, 5)]


# the nodes refuse a window wider than the channel count, like the reference (channel_pool.h:39)
WINDOW_CASES = [(shape, nsize) for shape in WINDOW_SHAPES for nsize in (3, 5, 7) if nsize <= shape[1]]


def _window_case(shape, nsize, op):
    rng = np.random.default_rng(nsize * 100 + op + sum(shape))
    a = rng.standard_normal(shape).astype(f32)
    pooled = _chpool(a if op == 0 else a * a, nsize, 1, nsize // 2, "sum")
    return a, pooled if op == 0 else a * (pooled * f32(0.1) + f32(1))


@pytest.mark.parametrize("shape,nsize", WINDOW_CASES)
@pytest.mark.parametrize("op", [0, 19])
def test_channel_windows_on_host_tensors(host_lib, shape, nsize, op):
    a, want = _window_case(shape, nsize, op)
    out = np.full(want.shape, np.nan, f32)
    assert host_lib.host_extensions_f32(op, _ptr(out), _ptr(a), None, None, *shape, nsize, 0, 0) == 0
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32)), (op, shape, nsize)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,nsize", WINDOW_CASES)
@pytest.mark.parametrize("op", [0, 19])
def test_channel_windows_across_groups_of_planes(shape, nsize, op):
    import mshadow_amd
    G = mshadow_amd.load_cases()
    G.set_device(0)
    a, want = _window_case(shape, nsize, op)
    out = G.to_device(np.full(want.shape, np.nan, f32))
    G.case_extensions(op, out, G.to_device(a), None, None, *shape, nsize, 0, 0)
    assert np.array_equal(out.download().view(np.uint32), want.view(np.uint32)), (op, shape, nsize)


PERMUTE_CASES = [
    ((5, 7), (1, 0)), ((64, 64), (1, 0)), ((65, 130), (1, 0)), ((1, 9), (1, 0)),
    ((3, 4, 5), (2, 1, 0)), ((3, 4, 5), (1, 0, 2)), ((3, 4, 5), (0, 2, 1)), ((3, 4, 5), (2, 0, 1)),
    ((2, 3, 4, 8), (0, 2, 3, 1)), ((2, 3, 4, 8), (0, 3, 1, 2)), ((2, 3, 4, 8), (3, 2, 1, 0)),
    ((2, 3, 4, 8), (1, 0, 2, 3)), ((2, 3, 4, 8), (0, 1, 2, 3)), ((2, 1, 4, 1), (3, 2, 1, 0)),
    ((4, 16, 70, 3), (0, 2, 3, 1)), ((2, 3, 2, 5, 6), (4, 0, 3, 1, 2)), ((2, 2, 3, 2, 2, 5), (5, 4, 3, 2, 1, 0)),
    ((8, 100, 33, 9), (0, 3, 1, 2)), ((0, 4, 5), (2, 1, 0)),
    ((2, 68, 8, 12), (0, 2, 3, 1)), ((3, 128, 200), (0, 2, 1)), ((4, 8, 16, 12), (3, 1, 2, 0)),
    ((2, 4, 36, 4), (2, 0, 1, 3)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("shape,axes", PERMUTE_CASES)
@pytest.mark.parametrize("dtype", [np.float32, np.int32])
def test_permute_entry_point(shape, axes, dtype):
    """mshadow_hip_permute_32 against numpy.transpose: every element in its new place"""
    import mshadow_amd
    G = mshadow_amd.load_cases()
    G.set_device(0)
    a = np.arange(int(np.prod(shape)), dtype=np.int64).reshape(shape)
    a = (a * 2654435761 % 2**31).astype(dtype)       # every element distinct enough to notice a mix-up
    want = np.ascontiguousarray(a.transpose(axes))
    if a.size == 0:   # nothing to move: the call must succeed without touching memory
        src, out = G.buffer((1,), dtype), G.buffer((1,), dtype)
        src.shape = shape
        G.permute(out, src, axes)
        return
    out = G.to_device(np.full(want.shape, -1, dtype))
    G.permute(out, G.to_device(a), axes)
    assert np.array_equal(out.download(), want), (shape, axes)


@pytest.mark.gpu
@pytest.mark.parametrize("shape,pad", [((7, 13), 0), ((7, 13), 3), ((64, 256), 0), ((5, 8), 4), ((1, 1), 0),
                                       ((3, 4, 5, 8), 0)])
def test_fill_entry_point(shape, pad):
    """mshadow_hip_fill_32 sets exactly the elements of the view; the pitch gap keeps its contents"""
    import mshadow_amd
    G = mshadow_amd.load_cases()
    G.set_device(0)
    buf = G.buffer(shape, f32, pad=pad, fill=0)
    G.fill(buf, -1.5)
    assert np.array_equal(buf.download(), np.full(shape, -1.5, f32))
    if pad:
        raw = G.buffer((buf.rows, buf.stride), f32)
        G.check(G.dll.mshadow_hip_memcpy2d_async(raw.ptr, raw.stride * 4, buf.ptr, buf.stride * 4,
                                                 buf.stride * 4, buf.rows, 3, None))
        G.stream_sync(None)
        assert np.all(raw.download()[:, buf.cols:] == 0)
