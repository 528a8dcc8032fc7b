"""ctypes bindings for the two CPU checkers (test infrastructure only).

`Checker("orc")` is the plain-C restatement in oracle/liboracle.so; `Checker("ref")` is
the reference's own headers compiled into oracle/_ref/libmshadow_ref.so (present only
where it was built). Both export the same functions with a different prefix, so one
binding serves both. Arrays are numpy; a 2-D array's row pitch is taken from its strides,
which lets tests pass padded (stride != cols) views.
"""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_SO = os.path.join(ROOT, "oracle", "liboracle.so")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libmshadow_ref.so")

SAVETO, PLUSTO, MINUSTO, MULTO, DIVTO = range(5)
SUM, MAX, MIN = range(3)
GRAD_SMOOTH, GRAD_IGNORE = 1, 2

_i = C.c_int
_f = C.c_float
_p = C.c_void_p


def pitch(a):
    """Row pitch in elements of the 2-D view (rows = all leading dims, cols = last)."""
    assert a.strides[-1] == a.itemsize, "last dimension must be dense"
    if a.ndim == 1:
        return a.shape[0]
    st = a.strides[-2] // a.itemsize
    # leading dims must be dense over the pitched rows
    exp = st * a.itemsize
    for d in range(a.ndim - 2, -1, -1):
        assert a.strides[d] == exp, "not a pitched row-major layout"
        exp *= a.shape[d]
    return st


def ptr(a):
    return C.c_void_p(a.ctypes.data)


def padded(shape, dtype, pad, fill=None, rng=None):
    """Allocate a row-major array whose rows carry `pad` extra elements; return the view."""
    shape = tuple(shape)
    full = np.empty(shape[:-1] + (shape[-1] + pad,), dtype=dtype)
    if fill is not None:
        full[...] = fill
    return full[..., : shape[-1]]


class Checker:
    def __init__(self, prefix):
        path = {"orc": ORACLE_SO, "ref": REF_SO}[prefix]
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        self.lib = C.CDLL(path)
        self.prefix = prefix
        self._sig()

    def _fn(self, name, argtypes, restype=None):
        f = getattr(self.lib, f"{self.prefix}_{name}")
        f.argtypes = argtypes
        f.restype = restype
        setattr(self, "_" + name, f)

    def _sig(self):
        self._fn("num_threads", [], _i)
        self._fn("float2half_n", [_p, _p, C.c_int64])
        self._fn("half2float_n", [_p, _p, C.c_int64])
        self._fn("map_fused_f32", [_p, _i, _p, _i, _p, _i, _p, _i, _p, _i, _i, _i, _i])
        self._fn("map_scalar_f32", [_p, _i, _i, _i, _f, _i])
        self._fn("map_axpb_f32", [_p, _i, _p, _i, _i, _i, _f, _f, _f, _i])
        self._fn("reduce_keep_lowest_f32", [_p, _p, _i, _i, _i, _i, _i, _f])
        self._fn("reduce_keep_highdim_f32", [_p, _p, _i, _i, _i, _i, _i, _i, _i, _f])
        self._fn("softmax_f32", [_p, _i, _p, _i, _i, _i])
        self._fn("softmax_grad_f32", [_p, _i, _p, _i, _p, _i, _i])
        _h = C.c_uint16
        self._fn("reduce_keep_lowest_f16", [_p, _p, _i, _i, _i, _i, _i, _h])
        self._fn("reduce_keep_highdim_f16", [_p, _p, _i, _i, _i, _i, _i, _i, _i, _h])
        self._fn("map_muladd_f16", [_p, _i, _p, _i, _p, _i, _p, _i, _i, _i, _i])
        self._fn("pool_f16", [_p, _i, _p, _i] + [_i] * 10)
        self._fn("softmax_f16", [_p, _i, _p, _i, _i, _i])
        self._fn("softmax_grad_f16", [_p, _i, _p, _i, _p, _i, _i])
        self._fn("softmax_grad_ex_f32", [_p, _i, _p, _i, _p, _i, _i, _i, _f, _f])
        self._fn("softmax3d_f32", [_p, _i, _p, _i, _i, _i, _i])
        self._fn("softmax3d_grad_f32", [_p, _i, _p, _i, _p, _i, _i, _i, _i, _i, _f, _f])
        self._fn("add_take_grad_f32", [_p, _i, _i, _p, _i, _i, _p, _i, _i])
        self._fn("add_take_grad_large_batch_f32", [_p, _i, _p, _p, _i, _i, _p, _i, _i])
        self._fn("index_fill_f32", [_p, _i, _p, _i, _i, _p, _i, _i])
        self._fn("grad_family_any", [_i, _p, _i, _p, _i, _p, _i, _i, _i, _i, _i, C.c_double, _f])
        self._fn("softmax3d_any", [_i, _p, _i, _p, _i, _i, _i, _i])
        self._fn("rows_by_index_any", [_i, _i, _i, _p, _i, _i, _p, _p, _i, _p, _i, _i])
        self._fn("sort_by_key_32", [_p, _i, _p, _i, _i])
        self._fn("vectorized_sort_32", [_p, _i, _p, _i])
        if self.prefix == "ref":
            self._fn("sort_by_key_any", [_i, _i, _p, _p, _i, _i])
            self._fn("shaping_f32", [_i, _p, _p, _p, _i, _i, _i, _i])
            self._fn("extensions_f32", [_i, _p, _p, _p, _p] + [_i] * 7)
            self._fn("random_f32", [_i, _i, _p, _i, _f, _f])
            self._fn("dot_f32", [_i, _p, _p, _p, _i, _i, _i])
        self._fn("pool_f32", [_p, _i, _p, _i] + [_i] * 10)
        self._fn("unpool_f32", [_p, _i, _p, _i, _p, _i, _p, _i] + [_i] * 10)
        for t in ("f16", "f32"):
            self._fn(f"im2col_{t}", [_p, _i, _p, _i] + [_i] * 12)
            self._fn(f"col2im_{t}", [_p, _i, _p, _i] + [_i] * 12)

    # -- half
    def float2half(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape, dtype=np.uint16)
        self._float2half_n(ptr(out), ptr(x), x.size)
        return out

    def half2float(self, h):
        h = np.ascontiguousarray(h, dtype=np.uint16)
        out = np.empty(h.shape, dtype=np.float32)
        self._half2float_n(ptr(out), ptr(h), h.size)
        return out

    def num_threads(self):
        return self._num_threads()

    # -- map
    def map_fused(self, dst, a, b, c, d, saver=SAVETO):
        rows, cols = int(np.prod(dst.shape[:-1])), dst.shape[-1]
        self._map_fused_f32(ptr(dst), pitch(dst), ptr(a), pitch(a), ptr(b), pitch(b), ptr(c),
                            pitch(c), ptr(d), pitch(d), rows, cols, saver)
        return dst

    def map_scalar(self, dst, scalar, saver=SAVETO):
        rows, cols = int(np.prod(dst.shape[:-1])), dst.shape[-1]
        self._map_scalar_f32(ptr(dst), pitch(dst), rows, cols, scalar, saver)
        return dst

    def map_axpb(self, dst, a, s1, s2, s3, saver=SAVETO):
        rows, cols = int(np.prod(dst.shape[:-1])), dst.shape[-1]
        self._map_axpb_f32(ptr(dst), pitch(dst), ptr(a), pitch(a), rows, cols, s1, s2, s3, saver)
        return dst

    # -- reductions
    def reduce_keep_lowest(self, dst, src, reducer=SUM, saver=SAVETO, scale=1.0):
        rows, cols = int(np.prod(src.shape[:-1])), src.shape[-1]
        assert dst.shape == (cols,)
        if src.dtype == np.uint16:  # half_t tensors as their 16-bit patterns; scale is rounded to half
            self._reduce_keep_lowest_f16(ptr(dst), ptr(src), pitch(src), rows, cols, reducer, saver,
                                         int(self.float2half(np.array([scale], np.float32))[0]))
            return dst
        self._reduce_keep_lowest_f32(ptr(dst), ptr(src), pitch(src), rows, cols, reducer, saver,
                                     scale)
        return dst

    def reduce_keep_highdim(self, dst, src, reducer=SUM, saver=SAVETO, scale=1.0):
        n, c, y, x = src.shape
        assert dst.shape == (c,)
        if src.dtype == np.uint16:
            self._reduce_keep_highdim_f16(ptr(dst), ptr(src), pitch(src), n, c, y, x, reducer,
                                          saver, int(self.float2half(np.array([scale], np.float32))[0]))
            return dst
        self._reduce_keep_highdim_f32(ptr(dst), ptr(src), pitch(src), n, c, y, x, reducer, saver,
                                      scale)
        return dst

    # -- softmax
    def softmax(self, dst, src):
        rows, cols = src.shape
        if src.dtype == np.uint16:
            self._softmax_f16(ptr(dst), pitch(dst), ptr(src), pitch(src), rows, cols)
            return dst
        self._softmax_f32(ptr(dst), pitch(dst), ptr(src), pitch(src), rows, cols)
        return dst

    def softmax_grad(self, dst, src, label):
        rows, cols = src.shape
        if src.dtype == np.uint16:
            assert label.dtype == np.uint16 and label.shape == (rows,)
            self._softmax_grad_f16(ptr(dst), pitch(dst), ptr(src), pitch(src), ptr(label), rows, cols)
            return dst
        assert label.dtype == np.float32 and label.shape == (rows,)
        self._softmax_grad_f32(ptr(dst), pitch(dst), ptr(src), pitch(src), ptr(label), rows, cols)
        return dst

    def softmax_grad_ex(self, dst, src, label, flags, ignore_label=0.0, alpha=0.0):
        rows, cols = src.shape
        self._softmax_grad_ex_f32(ptr(dst), pitch(dst), ptr(src), pitch(src), ptr(label), rows,
                                  cols, flags, ignore_label, alpha)
        return dst

    def softmax3d(self, dst, src):
        d0, d1, d2 = src.shape
        self._softmax3d_f32(ptr(dst), pitch(dst), ptr(src), pitch(src), d0, d1, d2)
        return dst

    def softmax3d_grad(self, dst, src, label, flags, ignore_label=0.0, alpha=0.0):
        d0, d1, d2 = src.shape
        assert label.shape == (d0, d2)
        self._softmax3d_grad_f32(ptr(dst), pitch(dst), ptr(src), pitch(src), ptr(label),
                                 pitch(label), d0, d1, d2, flags, ignore_label, alpha)
        return dst

    @staticmethod
    def _is_int(index):
        assert index.dtype in (np.int32, np.float32)
        return 1 if index.dtype == np.int32 else 0

    def add_take_grad(self, dst, index, src):
        self._add_take_grad_f32(ptr(dst), pitch(dst), dst.shape[0], ptr(index), self._is_int(index),
                                index.shape[0], ptr(src), pitch(src), src.shape[1])
        return dst

    def add_take_grad_large_batch(self, dst, sorted_rows, index, src):
        assert sorted_rows.dtype == index.dtype
        self._add_take_grad_large_batch_f32(ptr(dst), pitch(dst), ptr(sorted_rows), ptr(index),
                                            self._is_int(index), index.shape[0], ptr(src),
                                            pitch(src), src.shape[1])
        return dst

    def index_fill(self, dst, index, src):
        self._index_fill_f32(ptr(dst), pitch(dst), ptr(index), self._is_int(index),
                             index.shape[0], ptr(src), pitch(src), src.shape[1])
        return dst

    TYPE_FLAG = {"float32": 0, "float64": 1, "float16": 2, "int32": 4, "int64": 6}

    def grad_family_any(self, dst, src, label, flags, ignore_label=0.0, alpha=0.0):
        """SoftmaxGrad / SmoothSoftmaxGrad (with or without ignore_label) on float32, float64
        or float16 (= half_t) arrays; 2-D or 3-D by src's shape"""
        if src.ndim == 2:
            d0, a, b = 0, src.shape[0], src.shape[1]
            lpitch = label.shape[0]
        else:
            d0, a, b = src.shape
            lpitch = pitch(label)
        self._grad_family_any(self.TYPE_FLAG[src.dtype.name], ptr(dst), pitch(dst), ptr(src),
                              pitch(src), ptr(label), lpitch, d0, a, b, flags, ignore_label, alpha)
        return dst

    def softmax3d_any(self, dst, src):
        d0, d1, d2 = src.shape
        self._softmax3d_any(self.TYPE_FLAG[src.dtype.name], ptr(dst), pitch(dst), ptr(src),
                            pitch(src), d0, d1, d2)
        return dst

    def rows_by_index_any(self, op, dst, sorted_rows, index, src):
        self._rows_by_index_any(op, self.TYPE_FLAG[dst.dtype.name], self.TYPE_FLAG[index.dtype.name],
                                ptr(dst), pitch(dst), dst.shape[0],
                                ptr(sorted_rows) if sorted_rows is not None else None, ptr(index),
                                index.shape[0], ptr(src), pitch(src), src.shape[1])
        return dst

    @staticmethod
    def _key_kind(keys):
        return {"float32": 0, "int32": 1, "uint32": 2}[keys.dtype.name]

    def sort_by_key_any(self, keys, values, is_ascend=True):
        """the reference's SortByKey<cpu> on arrays of any type of its type switch (ref only)"""
        flag = dict(self.TYPE_FLAG, uint8=3, int8=5)
        self._sort_by_key_any(flag[keys.dtype.name], flag[values.dtype.name], ptr(keys), ptr(values),
                              keys.shape[0], 1 if is_ascend else 0)
        return keys, values

    def sort_by_key(self, keys, values, is_ascend=True):
        """in place on two contiguous 1-D arrays of 32-bit elements"""
        self._sort_by_key_32(ptr(keys), self._key_kind(keys), ptr(values), keys.shape[0],
                             1 if is_ascend else 0)
        return keys, values

    def vectorized_sort(self, values, segments):
        self._vectorized_sort_32(ptr(values), self._key_kind(values), ptr(segments), values.shape[0])
        return values, segments

    def shaping(self, op, out, a, v, n, c, h, w):
        """reference build only: the index-remapping extension expressions"""
        self._shaping_f32(op, ptr(out), ptr(a), ptr(v), n, c, h, w)
        return out

    def random(self, op, seed, out, p0=0.0, p1=1.0):
        """reference build only: Random<cpu> samplers into a float vector"""
        self._random_f32(op, seed, ptr(out), out.shape[0], p0, p1)
        return out

    def dot(self, op, out, a, b, m, k, n):
        """reference build only: the matrix products it evaluates without an external BLAS
        (op 0..2 of the product cases)"""
        self._dot_f32(op, ptr(out), ptr(a), ptr(b), m, k, n)
        return out

    def extensions(self, op, out, a, b, c, n, ch, h, w, p0=0, p1=0, p2=0):
        """reference build only: channel pooling, axis, view and index look-up expressions"""
        self._extensions_f32(op, ptr(out), ptr(a), ptr(b) if b is not None else None,
                             ptr(c) if c is not None else None, n, ch, h, w, p0, p1, p2)
        return out

    # -- pool / unpool: arrays are (..., H, W); leading dims are planes
    def map_muladd_f16(self, dst, a, b, c, saver=SAVETO):
        rows, cols = int(np.prod(dst.shape[:-1])), dst.shape[-1]
        self._map_muladd_f16(ptr(dst), pitch(dst), ptr(a), pitch(a), ptr(b), pitch(b), ptr(c),
                             pitch(c), rows, cols, saver)
        return dst

    def pool(self, dst, src, ky, kx, sy, sx, reducer=MAX):
        h, w = src.shape[-2:]
        ph, pw = dst.shape[-2:]
        planes = int(np.prod(src.shape[:-2]))
        if src.dtype == np.uint16:
            self._pool_f16(ptr(dst), pitch(dst), ptr(src), pitch(src), planes, h, w, ph, pw, ky,
                           kx, sy, sx, reducer)
            return dst
        self._pool_f32(ptr(dst), pitch(dst), ptr(src), pitch(src), planes, h, w, ph, pw, ky, kx,
                       sy, sx, reducer)
        return dst

    def unpool(self, dst, src, pooled, grad, ky, kx, sy, sx, reducer=MAX):
        h, w = src.shape[-2:]
        ph, pw = pooled.shape[-2:]
        planes = int(np.prod(src.shape[:-2]))
        self._unpool_f32(ptr(dst), pitch(dst), ptr(src), pitch(src), ptr(pooled), pitch(pooled),
                         ptr(grad), pitch(grad), planes, h, w, ph, pw, ky, kx, sy, sx, reducer)
        return dst

    # -- im2col / col2im; img is (N, C, H, W), col is (ky*kx*C, OH*OW*N)
    @staticmethod
    def col_shape(n, c, h, w, ky, kx, sy, sx, dy, dx, pad_y, pad_x):
        hp, wp = h + 2 * pad_y, w + 2 * pad_x
        oh = (hp - (dy * (ky - 1) + 1)) // sy + 1
        ow = (wp - (dx * (kx - 1) + 1)) // sx + 1
        return (ky * kx * c, oh * ow * n)

    def im2col(self, col, img, ky, kx, sy, sx, dy=1, dx=1, pad_y=0, pad_x=0):
        n, c, h, w = img.shape
        t = "f16" if img.dtype == np.uint16 else "f32"
        assert col.shape == self.col_shape(n, c, h, w, ky, kx, sy, sx, dy, dx, pad_y, pad_x)
        getattr(self, f"_im2col_{t}")(ptr(col), pitch(col), ptr(img), pitch(img), n, c, h, w, ky,
                                      kx, sy, sx, dy, dx, pad_y, pad_x)
        return col

    def col2im(self, img, col, ky, kx, sy, sx, dy=1, dx=1, pad_y=0, pad_x=0):
        n, c, h, w = img.shape
        t = "f16" if img.dtype == np.uint16 else "f32"
        assert col.shape == self.col_shape(n, c, h, w, ky, kx, sy, sx, dy, dx, pad_y, pad_x)
        getattr(self, f"_col2im_{t}")(ptr(img), pitch(img), ptr(col), pitch(col), n, c, h, w, ky,
                                      kx, sy, sx, dy, dx, pad_y, pad_x)
        return img


def have_ref():
    return os.path.exists(REF_SO)
