/*
 * TEST INFRASTRUCTURE - not part of the shipped library.
 *
 * Thin C entry points around the *real* dmlc/mshadow headers (included from
 * /root/reference through -I, never copied): each function wraps the caller's
 * buffers in Tensor<cpu> handles and evaluates the same expression a user of the
 * reference would write. The resulting library (oracle/_ref/libmshadow_ref.so)
 * checks the C restatement in oracle.c bit for bit and serves as the timed CPU
 * baseline. Signatures mirror oracle.h with the prefix ref_.
 */
#include <mshadow/tensor.h>
#include <mshadow/random.h>

#include <omp.h>
#include <stdint.h>

#include "../mshadow_amd/cases/portable_math.h"
/* a caller program written against <mshadow/tensor.h>: here that is the reference's */
#include "../mshadow_amd/cases/conv_net.h"

using namespace mshadow;
using namespace mshadow::expr;

namespace {

/* caller-side functor, same shape as guide/neuralnet/nnet.cu:14-18 */
struct sigmoid {
  MSHADOW_XINLINE static float Map(float a) { return pmath_sigmoid(a); }
};

template <typename T>
Tensor<cpu, 2, T> T2(const T *p, int rows, int cols, int stride) {
  return Tensor<cpu, 2, T>(const_cast<T *>(p), Shape2(rows, cols), stride, NULL);
}
template <typename T>
Tensor<cpu, 4, T> T4(const T *p, int n, int c, int h, int w, int stride) {
  return Tensor<cpu, 4, T>(const_cast<T *>(p), Shape4(n, c, h, w), stride, NULL);
}
template <typename T>
Tensor<cpu, 3, T> T3(const T *p, int a, int b, int c, int stride) {
  return Tensor<cpu, 3, T>(const_cast<T *>(p), Shape3(a, b, c), stride, NULL);
}
template <typename T>
Tensor<cpu, 1, T> T1(const T *p, int n) {
  return Tensor<cpu, 1, T>(const_cast<T *>(p), Shape1(n));
}

template <typename Dst, typename E>
void Assign(Dst dst, const E &e, int saver) {
  switch (saver) {
    case 0: dst = e; break;
    case 1: dst += e; break;
    case 2: dst -= e; break;
    case 3: dst *= e; break;
    default: dst /= e; break;
  }
}

template <typename Reducer, typename Src>
void ReduceHigh(Tensor<cpu, 1, float> dst, const Src &src, int saver, float scale) {
  switch (saver) {
    case 0: dst = scale * reduce_except_dim<1, Reducer>(src); break;
    case 1: dst += scale * reduce_except_dim<1, Reducer>(src); break;
    case 2: dst -= scale * reduce_except_dim<1, Reducer>(src); break;
    case 3: dst *= scale * reduce_except_dim<1, Reducer>(src); break;
    default: dst /= scale * reduce_except_dim<1, Reducer>(src); break;
  }
}

typedef half::half_t HalfT;
const HalfT *H(const uint16_t *p) { return reinterpret_cast<const HalfT *>(p); }
HalfT *H(uint16_t *p) { return reinterpret_cast<HalfT *>(p); }

template <typename Reducer, typename Src>
void ReduceHighHalf(Tensor<cpu, 1, HalfT> dst, const Src &src, int saver, HalfT scale) {
  switch (saver) {
    case 0: dst = scale * reduce_except_dim<1, Reducer>(src); break;
    case 1: dst += scale * reduce_except_dim<1, Reducer>(src); break;
    case 2: dst -= scale * reduce_except_dim<1, Reducer>(src); break;
    case 3: dst *= scale * reduce_except_dim<1, Reducer>(src); break;
    default: dst /= scale * reduce_except_dim<1, Reducer>(src); break;
  }
}

/* the gradient family and the row scatter functions of the reference for one element type */
template <typename T>
Tensor<cpu, 3, T> T3p(const T *p, int d0, int d1, int d2, int stride) {
  Tensor<cpu, 3, T> t(const_cast<T *>(p), Shape3(d0, d1, d2));
  t.stride_ = stride;
  return t;
}
template <typename DType>
void RefGradFamily(void *dst, int dstride, const void *src, int sstride, const void *label,
                   int lstride, int d0, int rows_or_d1, int cols_or_d2, int flags,
                   double ignore_label, float alpha) {
  const DType *s = static_cast<const DType *>(src), *l = static_cast<const DType *>(label);
  DType *d = static_cast<DType *>(dst);
  const DType ignore = DType(static_cast<float>(ignore_label));
  if (d0 == 0) {
    const int rows = rows_or_d1, cols = cols_or_d2;
    Tensor<cpu, 2, DType> D = T2(d, rows, cols, dstride), S = T2(s, rows, cols, sstride);
    Tensor<cpu, 1, DType> L = T1(l, rows);
    switch (flags) {
      case 0: SoftmaxGrad(D, S, L); break;
      case 1: SmoothSoftmaxGrad(D, S, L, alpha); break;
      case 2: SoftmaxGrad(D, S, L, ignore); break;
      default: SmoothSoftmaxGrad(D, S, L, ignore, alpha); break;
    }
  } else {
    const int d1 = rows_or_d1, d2 = cols_or_d2;
    Tensor<cpu, 3, DType> D = T3p(d, d0, d1, d2, dstride), S = T3p(s, d0, d1, d2, sstride);
    Tensor<cpu, 2, DType> L = T2(l, d0, d2, lstride);
    switch (flags) {
      case 0: SoftmaxGrad(D, S, L); break;
      case 1: SmoothSoftmaxGrad(D, S, L, alpha); break;
      case 2: SoftmaxGrad(D, S, L, ignore); break;
      default: SmoothSoftmaxGrad(D, S, L, ignore, alpha); break;
    }
  }
}
template <typename IndexType, typename DType>
void RefRowsByIndex(int op, void *dst, int dstride, int k_rows, const void *sorted, const void *index,
                    int n_index, const void *src, int sstride, int cols) {
  /* the row count of src is not used by the reference beyond the indices */
  Tensor<cpu, 2, DType> D = T2(static_cast<const DType *>(dst), k_rows, cols, dstride);
  Tensor<cpu, 2, DType> S = T2(static_cast<const DType *>(src), 1 << 30, cols, sstride);
  Tensor<cpu, 1, IndexType> I = T1(static_cast<const IndexType *>(index), n_index);
  if (op == 0) {
    S.shape_[0] = n_index;
    AddTakeGrad(D, I, S);
  } else if (op == 1) {
    AddTakeGradLargeBatch(D, T1(static_cast<const IndexType *>(sorted), n_index), I, S);
  } else {
    S.shape_[0] = n_index;
    IndexFill(D, I, S);
  }
}
template <typename DType>
void RefRowsByIndexOfIndex(int index_flag, int op, void *dst, int dstride, int k_rows,
                           const void *sorted, const void *index, int n_index, const void *src,
                           int sstride, int cols) {
  switch (index_flag) {
    case kFloat32: RefRowsByIndex<float, DType>(op, dst, dstride, k_rows, sorted, index, n_index, src, sstride, cols); break;
    case kFloat16: RefRowsByIndex<HalfT, DType>(op, dst, dstride, k_rows, sorted, index, n_index, src, sstride, cols); break;
    case kInt32: RefRowsByIndex<int, DType>(op, dst, dstride, k_rows, sorted, index, n_index, src, sstride, cols); break;
    default: RefRowsByIndex<int64_t, DType>(op, dst, dstride, k_rows, sorted, index, n_index, src, sstride, cols); break;
  }
}

}  // namespace

extern "C" {

int ref_num_threads(void) { return omp_get_max_threads(); }

void ref_float2half_n(uint16_t *dst, const float *src, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = half::half_t(src[i]).half_;
}
void ref_half2float_n(float *dst, const uint16_t *src, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = static_cast<float>(half::half_t::Binary(src[i]));
}

void ref_map_fused_f32(float *dst, int dstride, const float *a, int astride, const float *b,
                       int bstride, const float *c, int cstride, const float *d, int dstride_d,
                       int rows, int cols, int saver) {
  Tensor<cpu, 2, float> A = T2(a, rows, cols, astride), B = T2(b, rows, cols, bstride),
                        C = T2(c, rows, cols, cstride), D = T2(d, rows, cols, dstride_d);
  Assign(T2(dst, rows, cols, dstride), A * B + 0.5f * F<sigmoid>(C) - D, saver);
}

void ref_map_scalar_f32(float *dst, int dstride, int rows, int cols, float scalar, int saver) {
  Tensor<cpu, 2, float> o = T2(dst, rows, cols, dstride);
  switch (saver) {
    case 0: o = scalar; break;
    case 1: o += scalar; break;
    case 2: o -= scalar; break;
    case 3: o *= scalar; break;
    default: o /= scalar; break;
  }
}

void ref_map_axpb_f32(float *dst, int dstride, const float *a, int astride, int rows, int cols,
                      float s1, float s2, float s3, int saver) {
  Tensor<cpu, 2, float> A = T2(a, rows, cols, astride);
  Assign(T2(dst, rows, cols, dstride), (A + s1) / s2 + s3, saver);
}

void ref_reduce_keep_lowest_f32(float *dst, const float *src, int sstride, int rows, int cols,
                                int reducer, int saver, float scale) {
  Tensor<cpu, 2, float> S = T2(src, rows, cols, sstride);
  Tensor<cpu, 1, float> o = T1(dst, cols);
  /* reduce_except_dim<1> of a 2-D source keeps the lowest dimension
     (reduceto1d.h:92-100), the same engine sum_rows uses */
  if (reducer == 0) ReduceHigh<red::sum>(o, S, saver, scale);
  else if (reducer == 1) ReduceHigh<red::maximum>(o, S, saver, scale);
  else ReduceHigh<red::minimum>(o, S, saver, scale);
}

void ref_reduce_keep_highdim_f32(float *dst, const float *src, int sstride, int n, int c, int y,
                                 int x, int reducer, int saver, float scale) {
  Tensor<cpu, 4, float> S = T4(src, n, c, y, x, sstride);
  Tensor<cpu, 1, float> o = T1(dst, c);
  if (reducer == 0) ReduceHigh<red::sum>(o, S, saver, scale);
  else if (reducer == 1) ReduceHigh<red::maximum>(o, S, saver, scale);
  else ReduceHigh<red::minimum>(o, S, saver, scale);
}

void ref_softmax_f32(float *dst, int dstride, const float *src, int sstride, int rows, int cols) {
  Softmax(T2(dst, rows, cols, dstride), T2(src, rows, cols, sstride));
}

void ref_softmax_grad_f32(float *dst, int dstride, const float *src, int sstride,
                          const float *label, int rows, int cols) {
  SoftmaxGrad(T2(dst, rows, cols, dstride), T2(src, rows, cols, sstride), T1(label, rows));
}

/* the same on half_t tensors */
void ref_reduce_keep_lowest_f16(uint16_t *dst, const uint16_t *src, int sstride, int rows,
                                int cols, int reducer, int saver, uint16_t scale) {
  Tensor<cpu, 2, HalfT> S = T2(H(src), rows, cols, sstride);
  Tensor<cpu, 1, HalfT> o = T1(H(dst), cols);
  const HalfT sc = HalfT::Binary(scale);
  if (reducer == 0) ReduceHighHalf<red::sum>(o, S, saver, sc);
  else if (reducer == 1) ReduceHighHalf<red::maximum>(o, S, saver, sc);
  else ReduceHighHalf<red::minimum>(o, S, saver, sc);
}

void ref_reduce_keep_highdim_f16(uint16_t *dst, const uint16_t *src, int sstride, int n, int c,
                                 int y, int x, int reducer, int saver, uint16_t scale) {
  Tensor<cpu, 4, HalfT> S = T4(H(src), n, c, y, x, sstride);
  Tensor<cpu, 1, HalfT> o = T1(H(dst), c);
  const HalfT sc = HalfT::Binary(scale);
  if (reducer == 0) ReduceHighHalf<red::sum>(o, S, saver, sc);
  else if (reducer == 1) ReduceHighHalf<red::maximum>(o, S, saver, sc);
  else ReduceHighHalf<red::minimum>(o, S, saver, sc);
}

void ref_map_muladd_f16(uint16_t *dst, int dstride, const uint16_t *a, int astride,
                        const uint16_t *b, int bstride, const uint16_t *c, int cstride, int rows,
                        int cols, int saver) {
  Tensor<cpu, 2, HalfT> A = T2(H(a), rows, cols, astride), B = T2(H(b), rows, cols, bstride),
                        C = T2(H(c), rows, cols, cstride);
  Assign(T2(H(dst), rows, cols, dstride), A * B + C, saver);
}

void ref_pool_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride, int planes, int h,
                  int w, int ph, int pw, int ky, int kx, int sy, int sx, int reducer) {
  Tensor<cpu, 3, HalfT> S = T3(H(src), planes, h, w, sstride);
  Tensor<cpu, 3, HalfT> o = T3(H(dst), planes, ph, pw, dstride);
  if (reducer == 0) o = pool<red::sum>(S, Shape2(ph, pw), ky, kx, sy, sx);
  else if (reducer == 1) o = pool<red::maximum>(S, Shape2(ph, pw), ky, kx, sy, sx);
  else o = pool<red::minimum>(S, Shape2(ph, pw), ky, kx, sy, sx);
}

void ref_softmax_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride, int rows,
                     int cols) {
  Softmax(T2(H(dst), rows, cols, dstride), T2(H(src), rows, cols, sstride));
}

void ref_softmax_grad_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride,
                          const uint16_t *label, int rows, int cols) {
  SoftmaxGrad(T2(H(dst), rows, cols, dstride), T2(H(src), rows, cols, sstride),
              T1(H(label), rows));
}

void ref_softmax_grad_ex_f32(float *dst, int dstride, const float *src, int sstride,
                             const float *label, int rows, int cols, int flags,
                             float ignore_label, float alpha) {
  Tensor<cpu, 2, float> D = T2(dst, rows, cols, dstride), S = T2(src, rows, cols, sstride);
  Tensor<cpu, 1, float> L = T1(label, rows);
  switch (flags) {
    case 0: SoftmaxGrad(D, S, L); break;
    case 1: SmoothSoftmaxGrad(D, S, L, alpha); break;
    case 2: SoftmaxGrad(D, S, L, ignore_label); break;
    default: SmoothSoftmaxGrad(D, S, L, ignore_label, alpha); break;
  }
}

static Tensor<cpu, 3, float> T3s(const float *p, int d0, int d1, int d2, int stride) {
  Tensor<cpu, 3, float> t(const_cast<float *>(p), Shape3(d0, d1, d2));
  t.stride_ = stride;
  return t;
}

void ref_softmax3d_f32(float *dst, int dstride, const float *src, int sstride, int d0, int d1,
                       int d2) {
  Softmax(T3s(dst, d0, d1, d2, dstride), T3s(src, d0, d1, d2, sstride));
}

void ref_softmax3d_grad_f32(float *dst, int dstride, const float *src, int sstride,
                            const float *label, int lstride, int d0, int d1, int d2, int flags,
                            float ignore_label, float alpha) {
  Tensor<cpu, 3, float> D = T3s(dst, d0, d1, d2, dstride), S = T3s(src, d0, d1, d2, sstride);
  Tensor<cpu, 2, float> L = T2(label, d0, d2, lstride);
  switch (flags) {
    case 0: SoftmaxGrad(D, S, L); break;
    case 1: SmoothSoftmaxGrad(D, S, L, alpha); break;
    case 2: SoftmaxGrad(D, S, L, ignore_label); break;
    default: SmoothSoftmaxGrad(D, S, L, ignore_label, alpha); break;
  }
}

void ref_add_take_grad_f32(float *dst, int dstride, int k_rows, const void *index,
                           int index_is_int, int n_index, const float *src, int sstride,
                           int cols) {
  Tensor<cpu, 2, float> D = T2(dst, k_rows, cols, dstride), S = T2(src, n_index, cols, sstride);
  if (index_is_int) {
    AddTakeGrad(D, Tensor<cpu, 1, int>(const_cast<int *>(static_cast<const int *>(index)), Shape1(n_index)), S);
  } else {
    AddTakeGrad(D, T1(static_cast<const float *>(index), n_index), S);
  }
}

void ref_add_take_grad_large_batch_f32(float *dst, int dstride, const void *sorted,
                                       const void *index, int index_is_int, int n_index,
                                       const float *src, int sstride, int cols) {
  /* the row counts of dst and src are not used by the reference beyond the indices */
  Tensor<cpu, 2, float> D = T2(dst, 1 << 30, cols, dstride), S = T2(src, 1 << 30, cols, sstride);
  if (index_is_int) {
    AddTakeGradLargeBatch(D, Tensor<cpu, 1, int>(const_cast<int *>(static_cast<const int *>(sorted)), Shape1(n_index)),
                          Tensor<cpu, 1, int>(const_cast<int *>(static_cast<const int *>(index)), Shape1(n_index)), S);
  } else {
    AddTakeGradLargeBatch(D, T1(static_cast<const float *>(sorted), n_index),
                          T1(static_cast<const float *>(index), n_index), S);
  }
}

void ref_index_fill_f32(float *dst, int dstride, const void *index, int index_is_int,
                        int n_index, const float *src, int sstride, int cols) {
  Tensor<cpu, 2, float> D = T2(dst, 1 << 30, cols, dstride), S = T2(src, n_index, cols, sstride);
  if (index_is_int) {
    IndexFill(D, Tensor<cpu, 1, int>(const_cast<int *>(static_cast<const int *>(index)), Shape1(n_index)), S);
  } else {
    IndexFill(D, T1(static_cast<const float *>(index), n_index), S);
  }
}

void ref_grad_family_any(int type_flag, void *dst, int dstride, const void *src, int sstride,
                         const void *label, int lstride, int d0, int rows_or_d1, int cols_or_d2,
                         int flags, double ignore_label, float alpha) {
  MSHADOW_REAL_TYPE_SWITCH(type_flag, DType, {
    RefGradFamily<DType>(dst, dstride, src, sstride, label, lstride, d0, rows_or_d1, cols_or_d2,
                         flags, ignore_label, alpha);
  });
}

void ref_softmax3d_any(int type_flag, void *dst, int dstride, const void *src, int sstride, int d0,
                       int d1, int d2) {
  MSHADOW_REAL_TYPE_SWITCH(type_flag, DType, {
    Softmax(T3p(static_cast<const DType *>(dst), d0, d1, d2, dstride),
            T3p(static_cast<const DType *>(src), d0, d1, d2, sstride));
  });
}

void ref_rows_by_index_any(int op, int type_flag, int index_flag, void *dst, int dstride, int k_rows,
                           const void *sorted, const void *index, int n_index, const void *src,
                           int sstride, int cols) {
  MSHADOW_REAL_TYPE_SWITCH(type_flag, DType, {
    RefRowsByIndexOfIndex<DType>(index_flag, op, dst, dstride, k_rows, sorted, index, n_index, src,
                                 sstride, cols);
  });
}

/* key_kind 0: float keys with int values; 1: int keys with float values (the value words are
   only moved); uint32 keys are not a type the callers of the reference use */
void ref_sort_by_key_32(void *keys, int key_kind, void *values, int n, int is_ascend) {
  if (key_kind == 0) {
    SortByKey(Tensor<cpu, 1, float>(static_cast<float *>(keys), Shape1(n)),
              Tensor<cpu, 1, int>(static_cast<int *>(values), Shape1(n)), is_ascend != 0);
  } else {
    SortByKey(Tensor<cpu, 1, int>(static_cast<int *>(keys), Shape1(n)),
              Tensor<cpu, 1, float>(static_cast<float *>(values), Shape1(n)), is_ascend != 0);
  }
}
/* the reference's SortByKey<cpu> for any key / value type of its type switch */
void ref_sort_by_key_any(int key_flag, int value_flag, void *keys, void *values, int n,
                         int is_ascend) {
  MSHADOW_TYPE_SWITCH(key_flag, KDType, {
    MSHADOW_TYPE_SWITCH(value_flag, VDType, {
      SortByKey(Tensor<cpu, 1, KDType>(static_cast<KDType *>(keys), Shape1(n)),
                Tensor<cpu, 1, VDType>(static_cast<VDType *>(values), Shape1(n)), is_ascend != 0);
    });
  });
}
void ref_vectorized_sort_32(void *values, int value_kind, void *segments, int n) {
  Tensor<cpu, 1, int> seg(static_cast<int *>(segments), Shape1(n));
  if (value_kind == 0) VectorizedSort(Tensor<cpu, 1, float>(static_cast<float *>(values), Shape1(n)), seg);
  else VectorizedSort(Tensor<cpu, 1, int>(static_cast<int *>(values), Shape1(n)), seg);
}

/* index-remapping extensions (broadcast, repmat, reshape, swapaxis, mirror,
   upsampling_nearest): the same expressions the GPU cases library evaluates */
void ref_shaping_f32(int op, float *out, const float *a, const float *v, int n, int c, int h,
                     int w) {
#define OUT4(d0, d1, d2, d3) T4(out, d0, d1, d2, d3, d3)
#define OUT2(d0, d1) T2(out, d0, d1, d1)
#define IN4(d0, d1, d2, d3) T4(a, d0, d1, d2, d3, d3)
#define IN2(d0, d1) T2(a, d0, d1, d1)
#define VEC(len) T1(v, len)
  /* a: (n, c, h, w) contiguous input; v: c values; out: result, shape depends on op */
  switch (op) {
    case 0:   // bias add over channels, the convnet's `nhidden += broadcast<1>(hbias, shape)`
      OUT4(n, c, h, w) = IN4(n, c, h, w) + broadcast<1>(VEC(c), Shape4(n, c, h, w));
      break;
    case 1:   // row bias, `nout += repmat(obias, batch)` on the (n*c*h, w) view with w values
      OUT2(n * c * h, w) = IN2(n * c * h, w) + repmat(VEC(w), n * c * h);
      break;
    case 2:   // (c, n, h, w) -> (n, c, h, w), the convnet's conv forward epilogue
      OUT4(c, n, h, w) = swapaxis<1, 0>(reshape(IN2(n, c * h * w), Shape4(n, c, h, w)));
      break;
    case 3:   // the inverse direction, chained into a 2-D result
      OUT2(c, n * h * w) = reshape(swapaxis<1, 0>(IN4(n, c, h, w)), Shape2(c, n * h * w));
      break;
    case 4:   // swap the last dimension with the second
      OUT4(n, w, h, c) = swapaxis<3, 1>(IN4(n, c, h, w));
      break;
    case 5:   // swap two middle dimensions
      OUT4(n, h, c, w) = swapaxis<2, 1>(IN4(n, c, h, w));
      break;
    case 6:
      OUT4(n, c, h, w) = mirror(IN4(n, c, h, w));
      break;
    case 7:
      OUT4(n, c, h * 2, w * 2) = upsampling_nearest(IN4(n, c, h, w), 2);
      break;
    case 8:   // scalar broadcast scaled
      OUT4(n, c, h, w) = broadcast_scalar(VEC(1), Shape4(n, c, h, w)) * IN4(n, c, h, w);
      break;
    default:  // reshape of a vector expression
      OUT2(n * c, h * w) = reshape(VEC(n * c * h * w) * 2.0f, Shape2(n * c, h * w));
      break;
  }
#undef OUT4
#undef OUT2
#undef IN4
#undef IN2
#undef VEC
}

void ref_random_f32(int op, int seed, float *out, int n, float p0, float p1) {
#include "../mshadow_amd/cases/random_cases.inc"
}

/* caller-side functor of the extension cases (local response normalisation squares its input) */
struct square_of {
  MSHADOW_XINLINE static float Map(float a) { return a * a; }
};

void ref_extensions_f32(int op, float *out, const float *a, const float *b, const float *c, int n,
                        int ch, int h, int w, int p0, int p1, int p2) {
#define TENSOR(dim) Tensor<cpu, dim, float>
#define V1(p, len) T1(p, len)
#define V2(p, d0, d1) T2(p, d0, d1, d1)
#define V3(p, d0, d1, d2) T3(p, d0, d1, d2, d2)
#define V4(p, d0, d1, d2, d3) T4(p, d0, d1, d2, d3, d3)
#define V4S(p, d0, d1, d2, d3, pitch) T4(p, d0, d1, d2, d3, pitch)
#define MSHADOW_CASES_REFERENCE_HEADERS
#include "../mshadow_amd/cases/extension_cases.inc"
#undef MSHADOW_CASES_REFERENCE_HEADERS
#undef TENSOR
#undef V1
#undef V2
#undef V3
#undef V4S
#undef V4
}

/* the three matrix products the reference can evaluate without an external BLAS (its
   stand-alone build sends them to implicit_dot, dot_engine-inl.h:853-863); every other form
   of the product cases needs CBLAS or MKL there and is checked against float64 instead */
void ref_dot_f32(int op, float *out, const float *a, const float *b, int m, int k, int n) {
  const int batch = 1;
  (void)batch;
#define TENSOR(dim) Tensor<cpu, dim, float>
#define V2(p, d0, d1) T2(p, d0, d1, d1)
#define MSHADOW_CASES_REFERENCE_HEADERS
#include "../mshadow_amd/cases/dot_cases.inc"
#undef MSHADOW_CASES_REFERENCE_HEADERS
#undef TENSOR
#undef V2
}

void ref_pool_f32(float *dst, int dstride, const float *src, int sstride, int planes, int h, int w,
                  int ph, int pw, int ky, int kx, int sy, int sx, int reducer) {
  Tensor<cpu, 3, float> S = T3(src, planes, h, w, sstride);
  Tensor<cpu, 3, float> o = T3(dst, planes, ph, pw, dstride);
  if (reducer == 0) o = pool<red::sum>(S, Shape2(ph, pw), ky, kx, sy, sx);
  else if (reducer == 1) o = pool<red::maximum>(S, Shape2(ph, pw), ky, kx, sy, sx);
  else o = pool<red::minimum>(S, Shape2(ph, pw), ky, kx, sy, sx);
}

void ref_unpool_f32(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                    int pstride, const float *grad, int gstride, int planes, int h, int w, int ph,
                    int pw, int ky, int kx, int sy, int sx, int reducer) {
  Tensor<cpu, 3, float> S = T3(src, planes, h, w, sstride);
  Tensor<cpu, 3, float> P = T3(pooled, planes, ph, pw, pstride);
  Tensor<cpu, 3, float> G = T3(grad, planes, ph, pw, gstride);
  Tensor<cpu, 3, float> o = T3(dst, planes, h, w, dstride);
  if (reducer == 0) o = unpool<red::sum>(S, P, G, ky, kx, sy, sx);
  else if (reducer == 1) o = unpool<red::maximum>(S, P, G, ky, kx, sy, sx);
  else o = unpool<red::minimum>(S, P, G, ky, kx, sy, sx);
}

#define REF_IM2COL(NAME, CT, MT)                                                              \
  void NAME(CT *col, int cstride, const CT *img, int istride, int n, int c, int h, int w,     \
            int ky, int kx, int sy, int sx, int dy, int dx, int pad_y, int pad_x) {           \
    const int hp = h + 2 * pad_y, wp = w + 2 * pad_x;                                         \
    const int oh = (hp - (dy * (ky - 1) + 1)) / sy + 1, ow = (wp - (dx * (kx - 1) + 1)) / sx + 1; \
    Tensor<cpu, 4, MT> I = T4(reinterpret_cast<const MT *>(img), n, c, h, w, istride);        \
    Tensor<cpu, 2, MT> O = T2(reinterpret_cast<MT *>(col), ky * kx * c, oh * ow * n, cstride); \
    O = unpack_patch2col(pad(I, pad_y, pad_x), ky, kx, sy, sx, dy, dx);                       \
  }
REF_IM2COL(ref_im2col_f16, uint16_t, half::half_t)
REF_IM2COL(ref_im2col_f32, float, float)

#define REF_COL2IM(NAME, CT, MT)                                                              \
  void NAME(CT *img, int istride, const CT *col, int cstride, int n, int c, int h, int w,     \
            int ky, int kx, int sy, int sx, int dy, int dx, int pad_y, int pad_x) {           \
    const int hp = h + 2 * pad_y, wp = w + 2 * pad_x;                                         \
    const int oh = (hp - (dy * (ky - 1) + 1)) / sy + 1, ow = (wp - (dx * (kx - 1) + 1)) / sx + 1; \
    Tensor<cpu, 4, MT> I = T4(reinterpret_cast<MT *>(img), n, c, h, w, istride);              \
    Tensor<cpu, 2, MT> C = T2(reinterpret_cast<const MT *>(col), ky * kx * c, oh * ow * n, cstride); \
    I = crop(pack_col2patch(C, Shape4(n, c, hp, wp), ky, kx, sy, sx, dy, dx), Shape2(h, w),   \
             pad_y, pad_x);                                                                   \
  }
REF_COL2IM(ref_col2im_f16, uint16_t, half::half_t)
REF_COL2IM(ref_col2im_f32, float, float)

/* the convolutional network of cases/conv_net.h on the reference's CPU device (its stand-alone
   build evaluates the three forms of dot the program uses through implicit_dot) */
void ref_conv_net_f32(const int *v, int steps, float eta, float decay, const float *images,
                      const float *labels, const float *fixed_grad, float *kernel, float *weight,
                      float *const *keep) {
  const conv_net::Geometry g = {v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8]};
  conv_net::Train<cpu>(NULL, g, steps, eta, decay, images, labels, fixed_grad, kernel, weight, keep);
}

void ref_conv_pair(int half, const int *v, const void *image, const void *kernel,
                   const void *grad_out, void *col_forward, void *out, void *col_backward,
                   void *image_grad) {
  typedef half::half_t H;
  const conv_net::Geometry g = {v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8]};
  if (half) {
    conv_net::ConvPair<cpu, H>(NULL, g, static_cast<const H *>(image), static_cast<const H *>(kernel),
                               static_cast<const H *>(grad_out), static_cast<H *>(col_forward),
                               static_cast<H *>(out), static_cast<H *>(col_backward),
                               static_cast<H *>(image_grad));
  } else {
    conv_net::ConvPair<cpu, float>(NULL, g, static_cast<const float *>(image),
                                   static_cast<const float *>(kernel), static_cast<const float *>(grad_out),
                                   static_cast<float *>(col_forward), static_cast<float *>(out),
                                   static_cast<float *>(col_backward), static_cast<float *>(image_grad));
  }
}

}  // extern "C"
