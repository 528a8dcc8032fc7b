"""ctypes bindings of libmshadow_hip.so (include/mshadow_hip.h) and libmshadow_cases.so
(include/mshadow_hip_cases.h).

Nothing here computes: every operation is a call into the native library. Loading fails
loudly when the library has not been built (run `python -c "import __graft_entry__ as g;
g.build()"` or `python -m mshadow_amd.build`).
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
HIP_SO = os.path.join(HERE, "lib", "libmshadow_hip.so")
CASES_SO = os.path.join(HERE, "lib", "libmshadow_cases.so")

SAVETO, PLUSTO, MINUSTO, MULTO, DIVTO = range(5)
SUM, MAX, MIN = range(3)
H2D, D2H, D2D = 1, 2, 3
KEY_F32, KEY_I32, KEY_U32 = range(3)
BLAS_F32, BLAS_F64, BLAS_F16 = range(3)

_i, _f, _p, _sz = C.c_int, C.c_float, C.c_void_p, C.c_size_t
_d, _ll = C.c_double, C.c_longlong


class HipError(RuntimeError):
    pass


class Props(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_char * 64), ("compute_units", _i),
                ("wavefront_size", _i), ("max_threads_per_block", _i), ("clock_khz", _i),
                ("memory_clock_khz", _i), ("memory_bus_bits", _i), ("l2_bytes", _i),
                ("lds_bytes_per_block", _sz), ("total_global_mem", _sz)]


# name -> argtypes, for every symbol include/mshadow_hip.h and include/mshadow_hip_blas.h declare
HIP_SYMBOLS = {
    "mshadow_hip_last_error": ([], C.c_char_p),
    "mshadow_hip_abi_version": ([], _i),
    "mshadow_hip_device_count": ([C.POINTER(_i)], _i),
    "mshadow_hip_set_device": ([_i], _i),
    "mshadow_hip_get_device": ([C.POINTER(_i)], _i),
    "mshadow_hip_get_props": ([_i, C.POINTER(Props)], _i),
    "mshadow_hip_device_sync": ([], _i),
    "mshadow_hip_stream_create": ([C.POINTER(_p)], _i),
    "mshadow_hip_stream_destroy": ([_p], _i),
    "mshadow_hip_stream_sync": ([_p], _i),
    "mshadow_hip_stream_query": ([_p, C.POINTER(_i)], _i),
    "mshadow_hip_event_create": ([C.POINTER(_p)], _i),
    "mshadow_hip_event_destroy": ([_p], _i),
    "mshadow_hip_event_record": ([_p, _p], _i),
    "mshadow_hip_event_sync": ([_p], _i),
    "mshadow_hip_event_elapsed_ms": ([_p, _p, C.POINTER(_f)], _i),
    "mshadow_hip_malloc_pitch": ([C.POINTER(_p), C.POINTER(_sz), _sz, _sz], _i),
    "mshadow_hip_malloc": ([C.POINTER(_p), _sz], _i),
    "mshadow_hip_free": ([_p], _i),
    "mshadow_hip_malloc_host": ([C.POINTER(_p), _sz], _i),
    "mshadow_hip_free_host": ([_p], _i),
    "mshadow_hip_memcpy2d_async": ([_p, _sz, _p, _sz, _sz, _sz, _i, _p], _i),
    "mshadow_hip_memset_async": ([_p, _i, _sz, _p], _i),
    "mshadow_hip_launch": ([_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(_p), _sz,
                            _p], _i),
    "mshadow_hip_peek_last_error": ([], _i),
    "mshadow_hip_suggest_grid": ([_sz, _sz, _i, C.POINTER(C.c_uint32)], _i),
    "mshadow_hip_softmax_f32": ([_p, _i, _p, _i, _i, _i, _p], _i),
    "mshadow_hip_softmax_rowsum_f32": ([_p, _p, _i, _i, _i, _p], _i),
    "mshadow_hip_softmax_grad_ex_f32": ([_p, _i, _p, _i, _p, _i, _i, _i, _f, _f, _p], _i),
    "mshadow_hip_softmax3d_f32": ([_p, _i, _p, _i, _i, _i, _i, _p], _i),
    "mshadow_hip_softmax3d_grad_f32": ([_p, _i, _p, _i, _p, _i, _i, _i, _i, _i, _f, _f, _p], _i),
    "mshadow_hip_add_take_grad_f32": ([_p, _i, _i, _p, _i, _i, _p, _i, _i, _p], _i),
    "mshadow_hip_add_take_grad_large_batch_f32": ([_p, _i, _i, _p, _p, _i, _i, _p, _i, _i, _p], _i),
    "mshadow_hip_index_fill_f32": ([_p, _i, _i, _p, _i, _i, _p, _i, _i, _p], _i),
    "mshadow_hip_random_u32": ([_p, _sz, C.c_uint64, C.c_uint64, C.c_uint64, _p], _i),
    "mshadow_hip_random_uniform_f32": ([_p, _i, _i, _i, C.c_uint64, C.c_uint64, C.c_uint64, _f, _f, _p], _i),
    "mshadow_hip_random_normal_f32": ([_p, _i, _i, _i, C.c_uint64, C.c_uint64, C.c_uint64, _f, _f, _p], _i),
    "mshadow_hip_random_uniform_f64": ([_p, _i, _i, _i, C.c_uint64, C.c_uint64, C.c_uint64, C.c_double, C.c_double, _p], _i),
    "mshadow_hip_random_normal_f64": ([_p, _i, _i, _i, C.c_uint64, C.c_uint64, C.c_uint64, C.c_double, C.c_double, _p], _i),
    "mshadow_hip_fill_32": ([_p, _i, _i, _i, C.c_uint32, _p], _i),
    "mshadow_hip_fill_32_runs": ([_i, _i, _i, C.POINTER(C.c_int64), _i], _i),
    "mshadow_hip_reduce_scratch": ([_p, C.c_size_t, C.POINTER(_p), C.POINTER(_p)], _i),
    "mshadow_hip_permute_32": ([_p, _p, _i, C.POINTER(_i), C.POINTER(_i), _p], _i),
    "mshadow_hip_sort_by_key_workspace": ([_sz, C.POINTER(_sz)], _i),
    "mshadow_hip_sort_by_key_32": ([_p, _i, _p, _sz, _i, _p, _sz, _p], _i),
    "mshadow_hip_sort_by_key_32_noalloc": ([_p, _i, _p, _sz, _i, _p], _i),
    "mshadow_hip_graph_begin": ([_p], _i),
    "mshadow_hip_graph_end": ([_p, C.POINTER(C.c_void_p)], _i),
    "mshadow_hip_graph_launch": ([_p, _p], _i),
    "mshadow_hip_graph_destroy": ([_p], _i),
    "mshadow_hip_softmax_grad_f32": ([_p, _i, _p, _i, _p, _i, _i, _p], _i),
    "mshadow_hip_reduce_keep_lowest_f32": ([_p, _p, _i, _i, _i, _i, _i, _f, _p], _i),
    "mshadow_hip_reduce_keep_highdim_f32": ([_p, _p, _i, _i, _i, _i, _i, _i, _i, _f, _p], _i),
    "mshadow_hip_pool_f32": ([_p, _i, _p, _i] + [_i] * 10 + [_p], _i),
    "mshadow_hip_unpool_f32": ([_p, _i, _p, _i, _p, _i, _p, _i] + [_i] * 10 + [_p], _i),
    "mshadow_hip_im2col_f16": ([_p, _i, _p, _i] + [_i] * 12 + [_p], _i),
    "mshadow_hip_im2col_f32": ([_p, _i, _p, _i] + [_i] * 12 + [_p], _i),
    "mshadow_hip_col2im_f16": ([_p, _i, _p, _i] + [_i] * 12 + [_p], _i),
    "mshadow_hip_col2im_f32": ([_p, _i, _p, _i] + [_i] * 12 + [_p], _i),
    "mshadow_hip_blas_gemm": ([_i, _i, _i, _i, _i, _i, _d, _p, _i, _ll, _p, _i, _ll, _d, _p, _i, _ll, _i, _p], _i),
    "mshadow_hip_blas_gemv": ([_i, _i, _i, _i, _d, _p, _i, _ll, _p, _i, _ll, _d, _p, _i, _ll, _i, _p], _i),
    "mshadow_hip_blas_ger": ([_i, _i, _i, _d, _p, _i, _ll, _p, _i, _ll, _p, _i, _ll, _i, _p], _i),
    "mshadow_hip_blas_dot": ([_i, _i, _p, _i, _p, _i, _p, _p], _i),
}

CASES_SYMBOLS = {
    "mshadow_case_last_error": ([], C.c_char_p),
    "mshadow_case_map_fused_f32": ([_p, _i, _p, _i, _p, _i, _p, _i, _p, _i, _i, _i, _i, _p], _i),
    "mshadow_case_map_scalar_f32": ([_p, _i, _i, _i, _f, _i, _p], _i),
    "mshadow_case_map_axpb_f32": ([_p, _i, _p, _i, _i, _i, _f, _f, _f, _i, _p], _i),
    "mshadow_case_reduce_keep_lowest_f32": ([_p, _p, _i, _i, _i, _i, _i, _f, _i, _p], _i),
    "mshadow_case_reduce_keep_highdim_f32": ([_p, _p, _i, _i, _i, _i, _i, _i, _i, _f, _i, _p], _i),
    "mshadow_case_softmax_f32": ([_p, _i, _p, _i, _i, _i, _p], _i),
    "mshadow_case_reduce_keep_lowest_f16": ([_p, _p, _i, _i, _i, _i, _i, C.c_uint16, _i, _p], _i),
    "mshadow_case_reduce_keep_highdim_f16": ([_p, _p, _i, _i, _i, _i, _i, _i, _i, C.c_uint16, _i, _p], _i),
    "mshadow_case_softmax_f16": ([_p, _i, _p, _i, _i, _i, _p], _i),
    "mshadow_case_softmax_grad_f16": ([_p, _i, _p, _i, _p, _i, _i, _p], _i),
    "mshadow_case_softmax_f64": ([_p, _i, _p, _i, _i, _i, _p], _i),
    "mshadow_case_map_any": ([_i, _i, _p, _p, _p, _p, _i, _i, _p], _i),
    "mshadow_case_reduce_f64": ([_p, _p, _i, _i, _i, _i, _i, _i, C.c_double, _p], _i),
    "mshadow_case_map_muladd_f16": ([_p, _i, _p, _i, _p, _i, _p, _i, _i, _i, _i, _p], _i),
    "mshadow_case_pool_f16": ([_p, _i, _p, _i] + [_i] * 10 + [_p], _i),
    "mshadow_case_grad_family_f32": ([_p, _i, _p, _i, _p, _i, _i, _i, _i, _i, _f, _f, _p], _i),
    "mshadow_case_softmax3d_f32": ([_p, _i, _p, _i, _i, _i, _i, _p], _i),
    "mshadow_case_rows_by_index_f32": ([_i, _p, _i, _i, _p, _p, _i, _p, _i, _i, _i, _p], _i),
    "mshadow_case_grad_family_any": ([_i, _p, _i, _p, _i, _p, _i, _i, _i, _i, _i, C.c_double, _f, _p], _i),
    "mshadow_case_softmax3d_any": ([_i, _p, _i, _p, _i, _i, _i, _i, _p], _i),
    "mshadow_case_rows_by_index_any": ([_i, _i, _i, _p, _i, _i, _p, _p, _i, _p, _i, _i, _i, _p], _i),
    "mshadow_case_shaping_f32": ([_i, _p, _p, _p, _i, _i, _i, _i, _p], _i),
    "mshadow_case_random_f32": ([_i, _i, _p, _i, _f, _f, _p], _i),
    "mshadow_case_sort_by_key_any": ([_i, _i, _p, _p, _i, _i, _p], _i),
    "mshadow_case_random_f64": ([_i, _i, _p, _i, C.c_double, C.c_double, _p], _i),
    "mshadow_case_sort_by_key_32": ([_i, _p, _i, _p, _i, _i, _p], _i),
    "mshadow_case_extensions_f32": ([_i, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p], _i),
    "mshadow_case_dot_f32": ([_i, _p, _p, _p, _i, _i, _i, _i, _p], _i),
    "mshadow_case_half2_map": ([_p, _p, _i, _p], _i),
    "mshadow_case_two_layer_net_f32": ([_i, _f, _f, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p], _i),
    "mshadow_case_softmax_grad_f32": ([_p, _i, _p, _i, _p, _i, _i, _p], _i),
    "mshadow_case_pool_f32": ([_p, _i, _p, _i] + [_i] * 11 + [_p], _i),
    "mshadow_case_unpool_f32": ([_p, _i, _p, _i, _p, _i, _p, _i] + [_i] * 11 + [_p], _i),
    "mshadow_case_im2col_f16": ([_p, _i, _p, _i] + [_i] * 13 + [_p], _i),
    "mshadow_case_im2col_f32": ([_p, _i, _p, _i] + [_i] * 13 + [_p], _i),
    "mshadow_case_col2im_f16": ([_p, _i, _p, _i] + [_i] * 13 + [_p], _i),
    "mshadow_case_col2im_f32": ([_p, _i, _p, _i] + [_i] * 13 + [_p], _i),
    "mshadow_case_copy_roundtrip_f32": ([_p, _p, _i, _i, _i, C.POINTER(_i)], _i),
    "mshadow_case_copy_d2d_f32": ([_p, _i, _p, _i, _i, _i, _p], _i),
    "mshadow_case_conv_net_f32": ([_p, _i, _f, _f, _p, _p, _p, _p, _p, _p, _p], _i),
    "mshadow_case_conv_pair": ([_i, _p, _p, _p, _p, _p, _p, _p, _p, _p], _i),
}


def _bind(path, table):
    if not os.path.exists(path):
        raise HipError(f"{path} is not built; run `python -m mshadow_amd.build`")
    dll = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (argtypes, restype) in table.items():
        fn = getattr(dll, name)  # AttributeError if the symbol is not exported
        fn.argtypes = argtypes
        fn.restype = restype
    return dll


class DeviceBuffer:
    """A pitched 2-D allocation on the GPU holding an N-d array (rows = leading dims).

    `pad` adds that many unused elements to every row (stride = cols + pad), which is how
    tests exercise stride != cols. Uploads / downloads go through
    mshadow_hip_memcpy2d_async on the given stream.
    """

    def __init__(self, library, shape, dtype, pad=0, fill=None):
        self.lib = library
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.cols = self.shape[-1] if self.shape else 1
        self.rows = int(np.prod(self.shape[:-1])) if len(self.shape) > 1 else 1
        self.stride = self.cols + int(pad)
        self.nbytes = max(self.rows * self.stride * self.dtype.itemsize, 256)
        ptr = _p()
        library.check(library.dll.mshadow_hip_malloc(C.byref(ptr), self.nbytes))
        self.ptr = ptr.value
        if fill is not None:
            library.check(library.dll.mshadow_hip_memset_async(self.ptr, fill, self.nbytes, None))
            library.check(library.dll.mshadow_hip_stream_sync(None))

    @classmethod
    def from_array(cls, library, arr, pad=0, stream=None):
        buf = cls(library, arr.shape, arr.dtype, pad)
        buf.upload(arr, stream)
        return buf

    def upload(self, arr, stream=None):
        arr = np.ascontiguousarray(arr, dtype=self.dtype)
        assert arr.shape == self.shape, (arr.shape, self.shape)
        it = self.dtype.itemsize
        self.lib.check(self.lib.dll.mshadow_hip_memcpy2d_async(
            self.ptr, self.stride * it, arr.ctypes.data, self.cols * it, self.cols * it,
            self.rows, H2D, stream))
        self.lib.check(self.lib.dll.mshadow_hip_stream_sync(stream))

    def download(self, stream=None):
        out = np.empty(self.shape, dtype=self.dtype)
        it = self.dtype.itemsize
        self.lib.check(self.lib.dll.mshadow_hip_memcpy2d_async(
            out.ctypes.data, self.cols * it, self.ptr, self.stride * it, self.cols * it,
            self.rows, D2H, stream))
        self.lib.check(self.lib.dll.mshadow_hip_stream_sync(stream))
        return out

    def free(self):
        if self.ptr:
            self.lib.check(self.lib.dll.mshadow_hip_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Library:
    """Loaded libmshadow_hip.so (+ optionally libmshadow_cases.so) with error checking."""

    def __init__(self, with_cases=False):
        self.dll = _bind(HIP_SO, HIP_SYMBOLS)
        self.cases = _bind(CASES_SO, CASES_SYMBOLS) if with_cases else None

    # -- status handling
    def check(self, status):
        if status != 0:
            raise HipError(self.dll.mshadow_hip_last_error().decode(errors="replace"))

    def check_case(self, status):
        if status != 0:
            raise HipError(self.cases.mshadow_case_last_error().decode(errors="replace"))

    # -- runtime
    def device_count(self):
        n = _i(0)
        self.check(self.dll.mshadow_hip_device_count(C.byref(n)))
        return n.value

    def set_device(self, dev):
        self.check(self.dll.mshadow_hip_set_device(dev))

    def props(self, dev=0):
        p = Props()
        self.check(self.dll.mshadow_hip_get_props(dev, C.byref(p)))
        return p

    def stream_create(self):
        s = _p()
        self.check(self.dll.mshadow_hip_stream_create(C.byref(s)))
        return s.value

    def stream_destroy(self, s):
        self.check(self.dll.mshadow_hip_stream_destroy(s))

    def stream_sync(self, s=None):
        self.check(self.dll.mshadow_hip_stream_sync(s))

    def device_sync(self):
        self.check(self.dll.mshadow_hip_device_sync())

    # -- a sequence of launches recorded once and replayed
    def graph_begin(self, stream):
        self.check(self.dll.mshadow_hip_graph_begin(stream))

    def graph_end(self, stream):
        g = C.c_void_p()
        self.check(self.dll.mshadow_hip_graph_end(stream, C.byref(g)))
        return g

    def graph_launch(self, graph, stream=None):
        self.check(self.dll.mshadow_hip_graph_launch(graph, stream))

    def graph_destroy(self, graph):
        self.check(self.dll.mshadow_hip_graph_destroy(graph))

    def event_create(self):
        e = _p()
        self.check(self.dll.mshadow_hip_event_create(C.byref(e)))
        return e.value

    def event_destroy(self, e):
        self.check(self.dll.mshadow_hip_event_destroy(e))

    def event_record(self, e, s):
        self.check(self.dll.mshadow_hip_event_record(e, s))

    def event_sync(self, e):
        self.check(self.dll.mshadow_hip_event_sync(e))

    def elapsed_ms(self, start, stop):
        ms = _f(0)
        self.check(self.dll.mshadow_hip_event_elapsed_ms(start, stop, C.byref(ms)))
        return ms.value

    def buffer(self, shape, dtype, pad=0, fill=None):
        return DeviceBuffer(self, shape, dtype, pad, fill)

    def to_device(self, arr, pad=0, stream=None):
        return DeviceBuffer.from_array(self, arr, pad, stream)

    # -- fixed-function ops (DeviceBuffer arguments)
    def softmax(self, dst, src, stream=None):
        rows, cols = src.rows, src.cols
        self.check(self.dll.mshadow_hip_softmax_f32(dst.ptr, dst.stride, src.ptr, src.stride, rows,
                                                    cols, stream))

    def softmax_rowsum(self, sums, terms, stream=None):
        self.check(self.dll.mshadow_hip_softmax_rowsum_f32(sums.ptr, terms.ptr, terms.stride,
                                                           terms.rows, terms.cols, stream))

    def softmax_grad_ex(self, dst, src, label, flags, ignore_label=0.0, alpha=0.0, stream=None):
        self.check(self.dll.mshadow_hip_softmax_grad_ex_f32(
            dst.ptr, dst.stride, src.ptr, src.stride, label.ptr, src.rows, src.cols, flags,
            ignore_label, alpha, stream))

    def softmax3d(self, dst, src, stream=None):
        d0, d1, d2 = src.shape
        self.check(self.dll.mshadow_hip_softmax3d_f32(dst.ptr, dst.stride, src.ptr, src.stride,
                                                      d0, d1, d2, stream))

    def softmax3d_grad(self, dst, src, label, flags, ignore_label=0.0, alpha=0.0, stream=None):
        d0, d1, d2 = src.shape
        self.check(self.dll.mshadow_hip_softmax3d_grad_f32(
            dst.ptr, dst.stride, src.ptr, src.stride, label.ptr, label.stride, d0, d1, d2, flags,
            ignore_label, alpha, stream))

    @staticmethod
    def _index_is_int(index):
        assert index.dtype in (np.dtype(np.int32), np.dtype(np.float32))
        return 1 if index.dtype == np.dtype(np.int32) else 0

    def add_take_grad(self, dst, index, src, stream=None):
        self.check(self.dll.mshadow_hip_add_take_grad_f32(
            dst.ptr, dst.stride, dst.rows, index.ptr, self._index_is_int(index), index.cols,
            src.ptr, src.stride, src.cols, stream))

    def add_take_grad_large_batch(self, dst, sorted_rows, index, src, stream=None):
        self.check(self.dll.mshadow_hip_add_take_grad_large_batch_f32(
            dst.ptr, dst.stride, dst.rows, sorted_rows.ptr, index.ptr, self._index_is_int(index),
            index.cols, src.ptr, src.stride, src.cols, stream))

    def index_fill(self, dst, index, src, stream=None):
        self.check(self.dll.mshadow_hip_index_fill_f32(
            dst.ptr, dst.stride, dst.rows, index.ptr, self._index_is_int(index), index.cols,
            src.ptr, src.stride, src.cols, stream))

    def random_u32(self, dst, seed, subsequence=0, counter=0, stream=None):
        self.check(self.dll.mshadow_hip_random_u32(dst.ptr, dst.cols, seed, subsequence, counter, stream))

    def random_uniform(self, dst, seed, subsequence=0, counter=0, a=0.0, b=1.0, stream=None):
        """float32 or float64 buffers (the _f32 / _f64 entry point by the buffer's type)"""
        fn = (self.dll.mshadow_hip_random_uniform_f64 if dst.dtype == np.float64
              else self.dll.mshadow_hip_random_uniform_f32)
        self.check(fn(dst.ptr, dst.stride, dst.rows, dst.cols, seed, subsequence, counter, a, b, stream))

    def random_normal(self, dst, seed, subsequence=0, counter=0, mu=0.0, sigma=1.0, stream=None):
        fn = (self.dll.mshadow_hip_random_normal_f64 if dst.dtype == np.float64
              else self.dll.mshadow_hip_random_normal_f32)
        self.check(fn(dst.ptr, dst.stride, dst.rows, dst.cols, seed, subsequence, counter, mu, sigma, stream))

    def fill(self, dst, value, stream=None):
        """every element of a buffer of 32-bit elements set to `value`"""
        bits = int(np.array([value], dtype=dst.dtype).view(np.uint32)[0])
        self.check(self.dll.mshadow_hip_fill_32(dst.ptr, dst.stride, dst.rows, dst.cols, bits, stream))

    def permute(self, dst, src, axes, stream=None):
        """dst axis i = src axis axes[i]; dense buffers of 32-bit elements"""
        nd = len(src.shape)
        shape = (_i * nd)(*src.shape)
        ax = (_i * nd)(*axes)
        self.check(self.dll.mshadow_hip_permute_32(dst.ptr, src.ptr, nd, shape, ax, stream))

    @staticmethod
    def _key_kind(buf):
        return {"float32": KEY_F32, "int32": KEY_I32, "uint32": KEY_U32}[buf.dtype.name]

    def sort_by_key(self, keys, values, is_ascend=True, stream=None):
        """in place; the scratch buffer is allocated here and freed once the sort has finished"""
        n = keys.cols
        need = _sz(0)
        self.check(self.dll.mshadow_hip_sort_by_key_workspace(n, C.byref(need)))
        work = self.buffer((max(need.value, 1),), np.uint8)
        self.check(self.dll.mshadow_hip_sort_by_key_32(keys.ptr, self._key_kind(keys), values.ptr, n,
                                                       1 if is_ascend else 0, work.ptr, need.value,
                                                       stream))
        self.check(self.dll.mshadow_hip_stream_sync(stream))
        return need.value

    def sort_by_key_noalloc(self, keys, values, is_ascend=True, stream=None):
        """in place, at most SORT_NOALLOC_MAX pairs; the scratch memory is the library's own"""
        self.check(self.dll.mshadow_hip_sort_by_key_32_noalloc(
            keys.ptr, self._key_kind(keys), values.ptr, keys.cols, 1 if is_ascend else 0, stream))
        self.check(self.dll.mshadow_hip_stream_sync(stream))

    def softmax_grad(self, dst, src, label, stream=None):
        self.check(self.dll.mshadow_hip_softmax_grad_f32(dst.ptr, dst.stride, src.ptr, src.stride,
                                                         label.ptr, src.rows, src.cols, stream))

    def reduce_keep_lowest(self, dst, src, reducer=SUM, saver=SAVETO, scale=1.0, stream=None):
        self.check(self.dll.mshadow_hip_reduce_keep_lowest_f32(
            dst.ptr, src.ptr, src.stride, src.rows, src.cols, reducer, saver, scale, stream))

    def reduce_keep_highdim(self, dst, src, reducer=SUM, saver=SAVETO, scale=1.0, stream=None):
        n, c, y, x = src.shape
        self.check(self.dll.mshadow_hip_reduce_keep_highdim_f32(
            dst.ptr, src.ptr, src.stride, n, c, y, x, reducer, saver, scale, stream))

    def pool(self, dst, src, ky, kx, sy, sx, reducer=MAX, stream=None):
        h, w = src.shape[-2:]
        ph, pw = dst.shape[-2:]
        planes = int(np.prod(src.shape[:-2]))
        self.check(self.dll.mshadow_hip_pool_f32(dst.ptr, dst.stride, src.ptr, src.stride, planes,
                                                 h, w, ph, pw, ky, kx, sy, sx, reducer, stream))

    def unpool(self, dst, src, pooled, grad, ky, kx, sy, sx, reducer=MAX, stream=None):
        h, w = src.shape[-2:]
        ph, pw = pooled.shape[-2:]
        planes = int(np.prod(src.shape[:-2]))
        self.check(self.dll.mshadow_hip_unpool_f32(
            dst.ptr, dst.stride, src.ptr, src.stride, pooled.ptr, pooled.stride, grad.ptr,
            grad.stride, planes, h, w, ph, pw, ky, kx, sy, sx, reducer, stream))

    def im2col(self, col, img, ky, kx, sy, sx, dy=1, dx=1, pad_y=0, pad_x=0, stream=None):
        n, c, h, w = img.shape
        fn = self.dll.mshadow_hip_im2col_f16 if img.dtype == np.uint16 else \
            self.dll.mshadow_hip_im2col_f32
        self.check(fn(col.ptr, col.stride, img.ptr, img.stride, n, c, h, w, ky, kx, sy, sx, dy, dx,
                      pad_y, pad_x, stream))

    def col2im(self, img, col, ky, kx, sy, sx, dy=1, dx=1, pad_y=0, pad_x=0, stream=None):
        n, c, h, w = img.shape
        fn = self.dll.mshadow_hip_col2im_f16 if img.dtype == np.uint16 else \
            self.dll.mshadow_hip_col2im_f32
        self.check(fn(img.ptr, img.stride, col.ptr, col.stride, n, c, h, w, ky, kx, sy, sx, dy, dx,
                      pad_y, pad_x, stream))

    # -- caller-style programs through the C++ expression API (libmshadow_cases)
    def case_map_fused(self, dst, a, b, c, d, saver=SAVETO, stream=None):
        self.check_case(self.cases.mshadow_case_map_fused_f32(
            dst.ptr, dst.stride, a.ptr, a.stride, b.ptr, b.stride, c.ptr, c.stride, d.ptr,
            d.stride, dst.rows, dst.cols, saver, stream))

    def case_map_scalar(self, dst, scalar, saver=SAVETO, stream=None):
        self.check_case(self.cases.mshadow_case_map_scalar_f32(dst.ptr, dst.stride, dst.rows,
                                                               dst.cols, scalar, saver, stream))

    def case_copy_d2d(self, dst, src, stream=None, cols=None):
        """Copy(dst, src, stream) on device tensors; `cols` narrows both to their first columns"""
        self.check_case(self.cases.mshadow_case_copy_d2d_f32(
            dst.ptr, dst.stride, src.ptr, src.stride, dst.rows, dst.cols if cols is None else cols, stream))

    def case_map_axpb(self, dst, a, s1, s2, s3, saver=SAVETO, stream=None):
        self.check_case(self.cases.mshadow_case_map_axpb_f32(
            dst.ptr, dst.stride, a.ptr, a.stride, dst.rows, dst.cols, s1, s2, s3, saver, stream))

    def case_grad_family(self, dst, src, label, flags, ignore_label=0.0, alpha=0.0, stream=None):
        if len(src.shape) == 2:
            d0, a, b = 0, src.rows, src.cols
        else:
            d0, a, b = src.shape
        self.check_case(self.cases.mshadow_case_grad_family_f32(
            dst.ptr, dst.stride, src.ptr, src.stride, label.ptr, label.stride, d0, a, b, flags,
            ignore_label, alpha, stream))

    def case_softmax3d(self, dst, src, stream=None):
        d0, d1, d2 = src.shape
        self.check_case(self.cases.mshadow_case_softmax3d_f32(dst.ptr, dst.stride, src.ptr,
                                                              src.stride, d0, d1, d2, stream))

    def case_rows_by_index(self, op, dst, sorted_rows, index, src, stream=None):
        self.check_case(self.cases.mshadow_case_rows_by_index_f32(
            op, dst.ptr, dst.stride, dst.rows, sorted_rows.ptr if sorted_rows is not None else None,
            index.ptr, index.cols, src.ptr, src.stride, src.rows, src.cols, stream))

    # mshadow::TypeFlag codes of the element types the cases take (binary16 travels as float16)
    TYPE_FLAG = {"float32": 0, "float64": 1, "float16": 2, "int32": 4, "int64": 6}

    def case_grad_family_any(self, dst, src, label, flags, ignore_label=0.0, alpha=0.0, stream=None):
        """the four gradients on float / double / half_t tensors (2-D or 3-D by src's shape)"""
        if len(src.shape) == 2:
            d0, a, b = 0, src.rows, src.cols
        else:
            d0, a, b = src.shape
        self.check_case(self.cases.mshadow_case_grad_family_any(
            self.TYPE_FLAG[src.dtype.name], dst.ptr, dst.stride, src.ptr, src.stride, label.ptr,
            label.stride, d0, a, b, flags, ignore_label, alpha, stream))

    def case_softmax3d_any(self, dst, src, stream=None):
        d0, d1, d2 = src.shape
        self.check_case(self.cases.mshadow_case_softmax3d_any(
            self.TYPE_FLAG[src.dtype.name], dst.ptr, dst.stride, src.ptr, src.stride, d0, d1, d2, stream))

    def case_rows_by_index_any(self, op, dst, sorted_rows, index, src, stream=None):
        """op 0 AddTakeGrad, 1 AddTakeGradLargeBatch, 2 IndexFill for any table / index type"""
        self.check_case(self.cases.mshadow_case_rows_by_index_any(
            op, self.TYPE_FLAG[dst.dtype.name], self.TYPE_FLAG[index.dtype.name], dst.ptr, dst.stride,
            dst.rows, sorted_rows.ptr if sorted_rows is not None else None, index.ptr, index.cols,
            src.ptr, src.stride, src.rows, src.cols, stream))

    def case_sort_by_key_any(self, keys, values, is_ascend=True, stream=None):
        """SortByKey on buffers of any element type of the type switch"""
        flag = dict(self.TYPE_FLAG, uint8=3, int8=5)
        self.check_case(self.cases.mshadow_case_sort_by_key_any(
            flag[keys.dtype.name], flag[values.dtype.name], keys.ptr, values.ptr, keys.cols,
            1 if is_ascend else 0, stream))

    def case_shaping(self, op, out, a, v, n, c, h, w, stream=None):
        self.check_case(self.cases.mshadow_case_shaping_f32(op, out.ptr, a.ptr, v.ptr, n, c, h, w,
                                                            stream))

    # column-major BLAS entry points (include/mshadow_hip_blas.h); operands are DeviceBuffers
    def blas_gemm(self, dtype, transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc,
                  batch=1, strides=(0, 0, 0), stream=None):
        self.check(self.dll.mshadow_hip_blas_gemm(dtype, int(transa), int(transb), m, n, k, alpha,
                                                  A.ptr, lda, strides[0], B.ptr, ldb, strides[1],
                                                  beta, Cm.ptr, ldc, strides[2], batch, stream))

    def blas_gemv(self, dtype, trans, m, n, alpha, A, lda, x, incx, beta, y, incy, batch=1,
                  strides=(0, 0, 0), stream=None):
        self.check(self.dll.mshadow_hip_blas_gemv(dtype, int(trans), m, n, alpha, A.ptr, lda,
                                                  strides[0], x.ptr, incx, strides[1], beta,
                                                  y.ptr, incy, strides[2], batch, stream))

    def blas_ger(self, dtype, m, n, alpha, x, incx, y, incy, A, lda, batch=1, strides=(0, 0, 0),
                 stream=None):
        self.check(self.dll.mshadow_hip_blas_ger(dtype, m, n, alpha, x.ptr, incx, strides[0],
                                                 y.ptr, incy, strides[1], A.ptr, lda, strides[2],
                                                 batch, stream))

    def blas_dot(self, dtype, n, x, incx, y, incy, result, stream=None):
        self.check(self.dll.mshadow_hip_blas_dot(dtype, n, x.ptr, incx, y.ptr, incy, result.ptr,
                                                 stream))

    def case_random(self, op, seed, out, p0=0.0, p1=1.0, stream=None):
        fn = (self.cases.mshadow_case_random_f64 if out.dtype == np.float64
              else self.cases.mshadow_case_random_f32)
        self.check_case(fn(op, seed, out.ptr, out.cols, p0, p1, stream))

    def case_sort_by_key(self, op, keys, values, is_ascend=True, stream=None):
        self.check_case(self.cases.mshadow_case_sort_by_key_32(
            op, keys.ptr, self._key_kind(keys), values.ptr, keys.cols, 1 if is_ascend else 0,
            stream))

    def case_dot(self, op, out, a, b, m, k, n, batch=1, stream=None):
        self.check_case(self.cases.mshadow_case_dot_f32(op, out.ptr, a.ptr, b.ptr, m, k, n, batch, stream))

    def case_half2_map(self, out, x, stream=None):
        self.check_case(self.cases.mshadow_case_half2_map(out.ptr, x.ptr, x.cols // 2, stream))

    def case_two_layer_net(self, steps, eta, decay, x, label, w1, w2, probs, stream=None):
        """host numpy arrays (float32, contiguous); w1 and w2 are updated in place"""
        ptr = lambda a: a.ctypes.data_as(C.c_void_p)
        self.check_case(self.cases.mshadow_case_two_layer_net_f32(
            steps, eta, decay, x.shape[0], x.shape[1], w1.shape[1], w2.shape[1], ptr(x), ptr(label),
            ptr(w1), ptr(w2), ptr(probs), stream))

    def case_extensions(self, op, out, a, b, c, n, ch, h, w, p0=0, p1=0, p2=0, stream=None):
        self.check_case(self.cases.mshadow_case_extensions_f32(
            op, out.ptr, a.ptr, b.ptr if b is not None else None,
            c.ptr if c is not None else None, n, ch, h, w, p0, p1, p2, stream))

    def case_reduce_keep_lowest(self, dst, src, reducer=SUM, saver=SAVETO, scale=1.0, variant=0,
                                stream=None):
        """float tensors, or half_t tensors as uint16 buffers (scale then is the half's bits)"""
        fn = (self.cases.mshadow_case_reduce_keep_lowest_f16 if src.dtype == np.uint16
              else self.cases.mshadow_case_reduce_keep_lowest_f32)
        self.check_case(fn(dst.ptr, src.ptr, src.stride, src.rows, src.cols, reducer, saver, scale,
                           variant, stream))

    def case_reduce_keep_highdim(self, dst, src, reducer=SUM, saver=SAVETO, scale=1.0, variant=0,
                                 stream=None):
        n, c, y, x = src.shape
        fn = (self.cases.mshadow_case_reduce_keep_highdim_f16 if src.dtype == np.uint16
              else self.cases.mshadow_case_reduce_keep_highdim_f32)
        self.check_case(fn(dst.ptr, src.ptr, src.stride, n, c, y, x, reducer, saver, scale,
                           variant, stream))

    def case_softmax(self, dst, src, stream=None):
        fn = {"float32": self.cases.mshadow_case_softmax_f32,
              "uint16": self.cases.mshadow_case_softmax_f16,
              "float64": self.cases.mshadow_case_softmax_f64}[src.dtype.name]
        self.check_case(fn(dst.ptr, dst.stride, src.ptr, src.stride, src.rows, src.cols, stream))

    def case_softmax_grad(self, dst, src, label, stream=None):
        fn = (self.cases.mshadow_case_softmax_grad_f16 if src.dtype == np.uint16
              else self.cases.mshadow_case_softmax_grad_f32)
        self.check_case(fn(dst.ptr, dst.stride, src.ptr, src.stride, label.ptr, src.rows, src.cols,
                           stream))

    def case_reduce_f64(self, dst, src, reducer=SUM, scale=1.0, stream=None):
        """double tensors: a 2-D src keeps its columns, a 4-D src (n, c, y, x) keeps c"""
        if len(src.shape) == 2:
            n, c, (y, x) = 0, 0, src.shape
        else:
            n, c, y, x = src.shape
        self.check_case(self.cases.mshadow_case_reduce_f64(dst.ptr, src.ptr, src.stride, n, c, y, x,
                                                           reducer, scale, stream))

    def case_map_any(self, op, type_flag, dst, a, b, c, stream=None):
        """dense 2-D buffers of the element type the mshadow::TypeFlag code names"""
        self.check_case(self.cases.mshadow_case_map_any(op, type_flag, dst.ptr, a.ptr, b.ptr, c.ptr,
                                                        dst.rows, dst.cols, stream))

    def case_map_muladd_f16(self, dst, a, b, c, saver=SAVETO, stream=None):
        self.check_case(self.cases.mshadow_case_map_muladd_f16(
            dst.ptr, dst.stride, a.ptr, a.stride, b.ptr, b.stride, c.ptr, c.stride, dst.rows,
            dst.cols, saver, stream))

    def case_pool(self, dst, src, ky, kx, sy, sx, reducer=MAX, variant=0, stream=None):
        h, w = src.shape[-2:]
        ph, pw = dst.shape[-2:]
        planes = int(np.prod(src.shape[:-2]))
        if src.dtype == np.uint16:   # half_t tensors: the generic expression kernel
            self.check_case(self.cases.mshadow_case_pool_f16(
                dst.ptr, dst.stride, src.ptr, src.stride, planes, h, w, ph, pw, ky, kx, sy, sx,
                reducer, stream))
            return
        self.check_case(self.cases.mshadow_case_pool_f32(
            dst.ptr, dst.stride, src.ptr, src.stride, planes, h, w, ph, pw, ky, kx, sy, sx,
            reducer, variant, stream))

    def case_unpool(self, dst, src, pooled, grad, ky, kx, sy, sx, reducer=MAX, variant=0,
                    stream=None):
        h, w = src.shape[-2:]
        ph, pw = pooled.shape[-2:]
        planes = int(np.prod(src.shape[:-2]))
        self.check_case(self.cases.mshadow_case_unpool_f32(
            dst.ptr, dst.stride, src.ptr, src.stride, pooled.ptr, pooled.stride, grad.ptr,
            grad.stride, planes, h, w, ph, pw, ky, kx, sy, sx, reducer, variant, stream))

    def case_im2col(self, col, img, ky, kx, sy, sx, dy=1, dx=1, pad_y=0, pad_x=0, variant=0,
                    stream=None):
        n, c, h, w = img.shape
        fn = self.cases.mshadow_case_im2col_f16 if img.dtype == np.uint16 else \
            self.cases.mshadow_case_im2col_f32
        self.check_case(fn(col.ptr, col.stride, img.ptr, img.stride, n, c, h, w, ky, kx, sy, sx,
                           dy, dx, pad_y, pad_x, variant, stream))

    def case_col2im(self, img, col, ky, kx, sy, sx, dy=1, dx=1, pad_y=0, pad_x=0, variant=0,
                    stream=None):
        n, c, h, w = img.shape
        fn = self.cases.mshadow_case_col2im_f16 if img.dtype == np.uint16 else \
            self.cases.mshadow_case_col2im_f32
        self.check_case(fn(img.ptr, img.stride, col.ptr, col.stride, n, c, h, w, ky, kx, sy, sx,
                           dy, dx, pad_y, pad_x, variant, stream))

    def case_copy_roundtrip(self, arr, pad):
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        out = np.empty_like(arr)
        stride = _i(0)
        self.check_case(self.cases.mshadow_case_copy_roundtrip_f32(
            out.ctypes.data, arr.ctypes.data, arr.shape[0], arr.shape[1], int(pad),
            C.byref(stride)))
        return out, stride.value


class Probe:
    """libmshadow_probe.so: measurement aids of bench.py (csrc/mshadow_hip_probe.h)"""
    STAMPS = 16
    STAMP_ORDER = (10, 11, 12, 13, 1, 2, 6, 8, 3, 4, 5, 14)
    STAMP_NAMES = ("entry", "row loaded, thread maxima", "row maximum (barrier)", "exp",
                   "chunk sums and maxima exchanged (barrier)", "chunk plan",
                   "certain chunks quantised", "lists of the other chunks written",
                   "every wave's chunks done (barrier)", "row's list of addends assembled (barrier)",
                   "chain (wave 0; barrier)", "divided and stored (stores completed)")
    CHAIN_MODES = {"register": 0, "lds": 1, "lanes": 2, "register_f16": 3}

    def __init__(self):
        path = os.path.join(os.path.dirname(HIP_SO), "libmshadow_probe.so")
        if not os.path.exists(path):
            raise HipError(f"{path} is not built (python -m mshadow_amd.build)")
        self.dll = C.CDLL(path)
        self.dll.mshadow_probe_last_error.restype = C.c_char_p
        self.dll.mshadow_probe_add_chain.argtypes = [_i, _i, C.POINTER(C.c_double), _p]
        self.dll.mshadow_probe_softmax_phases.argtypes = [
            _p, _i, _p, _i, _i, _i, _i, C.POINTER(C.c_double), C.POINTER(C.c_double),
            C.POINTER(C.c_double), C.POINTER(_i), _p]

    def row_copy_us(self, dst, src, barriers, spin, stream=None, resident=2):
        us = C.c_double(0)
        self.dll.mshadow_probe_row_copy.argtypes = [_p, _i, _p, _i, _i, _i, _i, _i, _i, C.POINTER(C.c_double), _p]
        self._check(self.dll.mshadow_probe_row_copy(dst.ptr, dst.stride, src.ptr, src.stride, src.rows,
                                                    src.cols, barriers, spin, resident, C.byref(us), stream))
        return us.value

    def stream_copy_us(self, dst, src, floats, workgroups, own_run, stream=None):
        us = C.c_double(0)
        self.dll.mshadow_probe_stream_copy.argtypes = [_p, _p, C.c_size_t, _i, _i, C.POINTER(C.c_double), _p]
        self._check(self.dll.mshadow_probe_stream_copy(dst.ptr, src.ptr, floats, workgroups, int(own_run),
                                                       C.byref(us), stream))
        return us.value

    def row_copy_prefetch_us(self, dst, src, threads, prefetch_slabs, barriers, spin, workgroups, stream=None):
        us = C.c_double(0)
        self.dll.mshadow_probe_row_copy_prefetch.argtypes = [_p, _i, _p, _i, _i, _i, _i, _i, _i, _i, _i,
                                                             C.POINTER(C.c_double), _p]
        self._check(self.dll.mshadow_probe_row_copy_prefetch(
            dst.ptr, dst.stride, src.ptr, src.stride, src.rows, src.cols, threads, prefetch_slabs,
            barriers, spin, workgroups, C.byref(us), stream))
        return us.value

    def seg_rate_us(self, src, seg_len, nseg, segs, width, waves, piece_instr, stream=None):
        us = C.c_double(0)
        self.dll.mshadow_probe_seg_rate.argtypes = [_p, C.c_size_t, _i, _i, _i, _i, _i, _i,
                                                    C.POINTER(C.c_double), _p]
        self._check(self.dll.mshadow_probe_seg_rate(src.ptr, src.rows * src.stride, seg_len, nseg, segs,
                                                    width, waves, piece_instr, C.byref(us), stream))
        return us.value

    def highdim_split_us(self, dst, warm, src, config, stream=None):
        n, c, y, x = src.shape
        us = C.c_double(0)
        self.dll.mshadow_probe_highdim_split.argtypes = [_p, _p, _p, _i, _i, _i, _i, _i, C.POINTER(C.c_double), _p]
        self._check(self.dll.mshadow_probe_highdim_split(dst.ptr, warm.ptr, src.ptr, n, c, y, x, config,
                                                         C.byref(us), stream))
        return us.value

    def dma_rate_us(self, src, strip, width, waves, stream=None, window=32):
        """time to read `src` once by loads into LDS (strip 0/16/32 columns, width 4/16 bytes)"""
        us = C.c_double(0)
        self.dll.mshadow_probe_dma_rate.argtypes = [_p, _i, _i, _i, _i, _i, _i, _i, C.POINTER(C.c_double), _p]
        self._check(self.dll.mshadow_probe_dma_rate(src.ptr, src.stride, src.rows, src.cols, strip, width,
                                                    waves, window, C.byref(us), stream))
        return us.value

    def _check(self, status):
        if status != 0:
            raise HipError(self.dll.mshadow_probe_last_error().decode(errors="replace"))

    def add_chain_ns(self, mode, workgroups, stream=None):
        ns = C.c_double(0)
        self._check(self.dll.mshadow_probe_add_chain(self.CHAIN_MODES[mode], workgroups, C.byref(ns), stream))
        return ns.value

    def softmax_phases(self, dst, src, stream=None, variant=0):
        """-> ({step name: mean us since the previous step}, resident us, kernel us, fallback rows)"""
        mean = (C.c_double * self.STAMPS)()
        resident, kernel, fallback = C.c_double(0), C.c_double(0), _i(0)
        self._check(self.dll.mshadow_probe_softmax_phases(
            dst.ptr, dst.stride, src.ptr, src.stride, src.rows, src.cols, variant, mean, C.byref(resident),
            C.byref(kernel), C.byref(fallback), stream))
        steps = {f"{idx} {name}": mean[idx] for idx, name in zip(self.STAMP_ORDER, self.STAMP_NAMES)}
        return steps, resident.value, kernel.value, fallback.value


def load_probe():
    return Probe()


_lib = None
_cases = None


def load_lib():
    global _lib
    if _lib is None:
        _lib = Library(with_cases=False)
    return _lib


def load_cases():
    global _cases
    if _cases is None:
        _cases = Library(with_cases=True)
    return _cases


def lib():
    return load_lib()


def cases():
    return load_cases()
