/*
 * Caller-style programs against <mshadow/tensor.h>, exported as C (see
 * include/mshadow_hip_cases.h). Everything below is ordinary mshadow user code: handles
 * around existing memory, expressions, assignment. Built with DMLC_LOG_FATAL_THROW so a
 * failed CHECK comes back as an error code instead of aborting the test process.
 */
#define DMLC_LOG_FATAL_THROW 1
#include <mshadow/tensor.h>
#include <mshadow/random.h>
#include <mshadow_hip_cases.h>

#include <string>

#include "portable_math.h"
#include "two_layer_net.h"
#include "conv_net.h"

using namespace mshadow;
using namespace mshadow::expr;

namespace {

/* user functor, same shape as guide/neuralnet/nnet.cu:14-18 of the reference */
struct sigmoid {
  MSHADOW_XINLINE static float Map(float a) { return pmath_sigmoid(a); }
};

std::string &CaseError() {
  static thread_local std::string msg;
  return msg;
}

/* a Stream<gpu> object around a raw handle the caller owns */
struct BorrowedStream {
  Stream<gpu> s;
  explicit BorrowedStream(void *handle) { s.stream_ = handle; }
  Stream<gpu> *get() { return &s; }
};

template <typename T>
Tensor<gpu, 2, T> G2(const T *p, int rows, int cols, int stride, Stream<gpu> *s) {
  return Tensor<gpu, 2, T>(const_cast<T *>(p), Shape2(rows, cols), stride, s);
}
template <typename T>
Tensor<gpu, 3, T> G3(const T *p, int a, int b, int c, int stride, Stream<gpu> *s) {
  return Tensor<gpu, 3, T>(const_cast<T *>(p), Shape3(a, b, c), stride, s);
}
template <typename T>
Tensor<gpu, 4, T> G4(const T *p, int n, int c, int h, int w, int stride, Stream<gpu> *s) {
  return Tensor<gpu, 4, T>(const_cast<T *>(p), Shape4(n, c, h, w), stride, s);
}
template <typename T>
Tensor<gpu, 1, T> G1(const T *p, int n, Stream<gpu> *s) {
  return Tensor<gpu, 1, T>(const_cast<T *>(p), Shape1(n), s);
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

template <typename Reducer, typename DType, typename Src>
void ReduceInto(Tensor<gpu, 1, DType> dst, const Src &src, int saver, DType scale) {
  Assign(dst, scale * reduce_except_dim<1, Reducer>(src), saver);
}
template <typename DType, typename Src>
void ReduceDispatch(Tensor<gpu, 1, DType> dst, const Src &src, int reducer, int saver,
                    DType scale) {
  if (reducer == 0) ReduceInto<red::sum>(dst, src, saver, scale);
  else if (reducer == 1) ReduceInto<red::maximum>(dst, src, saver, scale);
  else ReduceInto<red::minimum>(dst, src, saver, scale);
}

typedef half::half_t HalfT;
inline const HalfT *H(const uint16_t *p) { return reinterpret_cast<const HalfT *>(p); }
inline HalfT *H(uint16_t *p) { return reinterpret_cast<HalfT *>(p); }

/* the gradient family and the row scatter functions for one element type (see the entry
   points mshadow_case_grad_family_any / mshadow_case_rows_by_index_any) */
template <typename DType>
void GradFamilyOf(void *dst, int dstride, const void *src, int sstride, const void *label,
                  int lstride, int d0, int rows_or_d1, int cols_or_d2, int flags,
                  double ignore_label, float alpha, Stream<gpu> *st) {
  const DType *s = static_cast<const DType *>(src), *l = static_cast<const DType *>(label);
  DType *d = static_cast<DType *>(dst);
  const DType ignore = DType(static_cast<float>(ignore_label));
  if (d0 == 0) {
    const int rows = rows_or_d1, cols = cols_or_d2;
    Tensor<gpu, 2, DType> D = G2(d, rows, cols, dstride, st), S = G2(s, rows, cols, sstride, st);
    Tensor<gpu, 1, DType> L = G1(l, rows, st);
    switch (flags) {
      case 0: SoftmaxGrad(D, S, L); break;
      case 1: SmoothSoftmaxGrad(D, S, L, alpha); break;
      case 2: SoftmaxGrad(D, S, L, ignore); break;
      default: SmoothSoftmaxGrad(D, S, L, ignore, alpha); break;
    }
  } else {
    const int d1 = rows_or_d1, d2 = cols_or_d2;
    Tensor<gpu, 3, DType> D = G3(d, d0, d1, d2, dstride, st), S = G3(s, d0, d1, d2, sstride, st);
    Tensor<gpu, 2, DType> L = G2(l, d0, d2, lstride, st);
    switch (flags) {
      case 0: SoftmaxGrad(D, S, L); break;
      case 1: SmoothSoftmaxGrad(D, S, L, alpha); break;
      case 2: SoftmaxGrad(D, S, L, ignore); break;
      default: SmoothSoftmaxGrad(D, S, L, ignore, alpha); break;
    }
  }
}
template <typename IndexType, typename DType>
void RowsByIndexOf(int op, void *dst, int dstride, int k_rows, const void *sorted, const void *index,
                   int n_index, const void *src, int sstride, int src_rows, int cols,
                   Stream<gpu> *st) {
  Tensor<gpu, 2, DType> D = G2(static_cast<const DType *>(dst), k_rows, cols, dstride, st);
  Tensor<gpu, 2, DType> S = G2(static_cast<const DType *>(src), src_rows, cols, sstride, st);
  Tensor<gpu, 1, IndexType> I = G1(static_cast<const IndexType *>(index), n_index, st);
  if (op == 0) {
    AddTakeGrad(D, I, S);
  } else if (op == 1) {
    AddTakeGradLargeBatch(D, G1(static_cast<const IndexType *>(sorted), n_index, st), I, S);
  } else {
    IndexFill(D, I, S);
  }
}
template <typename DType>
void RowsByIndexOfIndex(int index_flag, int op, void *dst, int dstride, int k_rows, const void *sorted,
                        const void *index, int n_index, const void *src, int sstride, int src_rows,
                        int cols, Stream<gpu> *st) {
  switch (index_flag) {
    case kFloat32:
      RowsByIndexOf<float, DType>(op, dst, dstride, k_rows, sorted, index, n_index, src, sstride, src_rows, cols, st);
      break;
    case kFloat16:
      RowsByIndexOf<HalfT, DType>(op, dst, dstride, k_rows, sorted, index, n_index, src, sstride, src_rows, cols, st);
      break;
    case kInt32:
      RowsByIndexOf<int, DType>(op, dst, dstride, k_rows, sorted, index, n_index, src, sstride, src_rows, cols, st);
      break;
    case kInt64:
      RowsByIndexOf<int64_t, DType>(op, dst, dstride, k_rows, sorted, index, n_index, src, sstride, src_rows, cols, st);
      break;
    default:
      LOG(FATAL) << "index type " << index_flag << " is not among the cases";
  }
}
}  // namespace

#define CASE_BEGIN try {
#define CASE_END                          \
  }                                       \
  catch (const std::exception &e) {       \
    CaseError() = e.what();               \
    return 1;                             \
  }                                       \
  return 0;

extern "C" {

const char *mshadow_case_last_error(void) { return CaseError().c_str(); }

int mshadow_case_map_fused_f32(float *dst, int dstride, const float *a, int astride,
                               const float *b, int bstride, const float *c, int cstride,
                               const float *d, int dstride_d, int rows, int cols, int saver,
                               void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 2, float> A = G2(a, rows, cols, astride, st.get()),
                        B = G2(b, rows, cols, bstride, st.get()),
                        C = G2(c, rows, cols, cstride, st.get()),
                        D = G2(d, rows, cols, dstride_d, st.get());
  Assign(G2(dst, rows, cols, dstride, st.get()), A * B + 0.5f * F<sigmoid>(C) - D, saver);
  CASE_END
}

int mshadow_case_map_scalar_f32(float *dst, int dstride, int rows, int cols, float scalar,
                                int saver, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 2, float> o = G2(dst, rows, cols, dstride, st.get());
  switch (saver) {
    case 0: o = scalar; break;
    case 1: o += scalar; break;
    case 2: o -= scalar; break;
    case 3: o *= scalar; break;
    default: o /= scalar; break;
  }
  CASE_END
}

int mshadow_case_map_axpb_f32(float *dst, int dstride, const float *a, int astride, int rows,
                              int cols, float s1, float s2, float s3, int saver, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 2, float> A = G2(a, rows, cols, astride, st.get());
  Assign(G2(dst, rows, cols, dstride, st.get()), (A + s1) / s2 + s3, saver);
  CASE_END
}

int mshadow_case_reduce_keep_lowest_f32(float *dst, const float *src, int sstride, int rows,
                                        int cols, int reducer, int saver, float scale,
                                        int variant, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 2, float> S = G2(src, rows, cols, sstride, st.get());
  Tensor<gpu, 1, float> o = G1(dst, cols, st.get());
  if (variant == 0) ReduceDispatch(o, S, reducer, saver, scale);
  else ReduceDispatch(o, F<op::identity>(S), reducer, saver, scale);
  CASE_END
}

int mshadow_case_reduce_keep_highdim_f32(float *dst, const float *src, int sstride, int n, int c,
                                         int y, int x, int reducer, int saver, float scale,
                                         int variant, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 4, float> S = G4(src, n, c, y, x, sstride, st.get());
  Tensor<gpu, 1, float> o = G1(dst, c, st.get());
  if (variant == 0) ReduceDispatch(o, S, reducer, saver, scale);
  else ReduceDispatch(o, F<op::identity>(S), reducer, saver, scale);
  CASE_END
}

int mshadow_case_softmax_f32(float *dst, int dstride, const float *src, int sstride, int rows,
                             int cols, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Softmax(G2(dst, rows, cols, dstride, st.get()), G2(src, rows, cols, sstride, st.get()));
  CASE_END
}

int mshadow_case_softmax_grad_f32(float *dst, int dstride, const float *src, int sstride,
                                  const float *label, int rows, int cols, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  SoftmaxGrad(G2(dst, rows, cols, dstride, st.get()), G2(src, rows, cols, sstride, st.get()),
              G1(label, rows, st.get()));
  CASE_END
}

/* the reductions and the softmax pair on half_t tensors (16-bit patterns; scale is a half_t) */
int mshadow_case_reduce_keep_lowest_f16(uint16_t *dst, const uint16_t *src, int sstride, int rows,
                                        int cols, int reducer, int saver, uint16_t scale,
                                        int variant, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 2, HalfT> S = G2(H(src), rows, cols, sstride, st.get());
  Tensor<gpu, 1, HalfT> o = G1(H(dst), cols, st.get());
  const HalfT sc = HalfT::Binary(scale);
  if (variant == 0) ReduceDispatch(o, S, reducer, saver, sc);
  else ReduceDispatch(o, F<op::identity>(S), reducer, saver, sc);
  CASE_END
}

int mshadow_case_reduce_keep_highdim_f16(uint16_t *dst, const uint16_t *src, int sstride, int n,
                                         int c, int y, int x, int reducer, int saver,
                                         uint16_t scale, int variant, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 4, HalfT> S = G4(H(src), n, c, y, x, sstride, st.get());
  Tensor<gpu, 1, HalfT> o = G1(H(dst), c, st.get());
  const HalfT sc = HalfT::Binary(scale);
  if (variant == 0) ReduceDispatch(o, S, reducer, saver, sc);
  else ReduceDispatch(o, F<op::identity>(S), reducer, saver, sc);
  CASE_END
}

int mshadow_case_softmax_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride,
                             int rows, int cols, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Softmax(G2(H(dst), rows, cols, dstride, st.get()), G2(H(src), rows, cols, sstride, st.get()));
  CASE_END
}

int mshadow_case_softmax_grad_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride,
                                  const uint16_t *label, int rows, int cols, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  SoftmaxGrad(G2(H(dst), rows, cols, dstride, st.get()), G2(H(src), rows, cols, sstride, st.get()),
              G1(H(label), rows, st.get()));
  CASE_END
}

/* dst <saver>= a * b + c and pool<Reducer> on half_t tensors (the generic expression kernels) */
int mshadow_case_map_muladd_f16(uint16_t *dst, int dstride, const uint16_t *a, int astride,
                                const uint16_t *b, int bstride, const uint16_t *c, int cstride,
                                int rows, int cols, int saver, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 2, HalfT> A = G2(H(a), rows, cols, astride, st.get()),
                        B = G2(H(b), rows, cols, bstride, st.get()),
                        C = G2(H(c), rows, cols, cstride, st.get());
  Assign(G2(H(dst), rows, cols, dstride, st.get()), A * B + C, saver);
  CASE_END
}

int mshadow_case_pool_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride, int planes,
                          int h, int w, int ph, int pw, int ky, int kx, int sy, int sx,
                          int reducer, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 3, HalfT> S = G3(H(src), planes, h, w, sstride, st.get());
  Tensor<gpu, 3, HalfT> o = G3(H(dst), planes, ph, pw, dstride, st.get());
  const Shape<2> ps = Shape2(ph, pw);
  if (reducer == 0) o = pool<red::sum>(S, ps, ky, kx, sy, sx);
  else if (reducer == 1) o = pool<red::maximum>(S, ps, ky, kx, sy, sx);
  else o = pool<red::minimum>(S, ps, ky, kx, sy, sx);
  CASE_END
}

/* dst = scale * reduce_except_dim<1, Reducer>(src) on double tensors: 2-D (n == 0: rows x cols =
   c x x... see the arguments) or 4-D (n, c, y, x) */
int mshadow_case_reduce_f64(double *dst, const double *src, int sstride, int n, int c, int y, int x,
                            int reducer, double scale, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  if (n == 0) {  // 2-D: y rows, x columns, keeps the columns
    Tensor<gpu, 2, double> S = G2(src, y, x, sstride, st.get());
    ReduceDispatch(G1(dst, x, st.get()), S, reducer, 0, scale);
  } else {
    Tensor<gpu, 4, double> S = G4(src, n, c, y, x, sstride, st.get());
    ReduceDispatch(G1(dst, c, st.get()), S, reducer, 0, scale);
  }
  CASE_END
}

/* dst = a * b + c on tensors of any element type of the type switch (mshadow::TypeFlag codes),
   and dst = pad(crop(a, (rows - 2, cols - 2)), 1) when op == 1: the generic expression kernels
   instantiated through MSHADOW_TYPE_SWITCH for every type it knows */
int mshadow_case_map_any(int op, int type_flag, void *dst, const void *a, const void *b,
                         const void *c, int rows, int cols, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  MSHADOW_TYPE_SWITCH(type_flag, DType, {
    Tensor<gpu, 2, DType> A = G2(static_cast<const DType *>(a), rows, cols, cols, st.get()),
                          B = G2(static_cast<const DType *>(b), rows, cols, cols, st.get()),
                          C = G2(static_cast<const DType *>(c), rows, cols, cols, st.get()),
                          D = G2(static_cast<const DType *>(dst), rows, cols, cols, st.get());
    if (op == 0) {
      D = A * B + C;
    } else {
      D = pad(crop(A, Shape2(rows - 2, cols - 2)), 1);
    }
  });
  CASE_END
}

/* Softmax(dst, src) on double tensors */
int mshadow_case_softmax_f64(double *dst, int dstride, const double *src, int sstride, int rows,
                             int cols, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Softmax(G2(dst, rows, cols, dstride, st.get()), G2(src, rows, cols, sstride, st.get()));
  CASE_END
}

/* the gradient family and the 3-D softmax through the C++ functions; flags as in
   mshadow_hip.h (bit 0 smooth, bit 1 ignore_label); d0 == 0 selects the 2-D functions */
int mshadow_case_grad_family_f32(float *dst, int dstride, const float *src, int sstride,
                                 const float *label, int lstride, int d0, int rows_or_d1,
                                 int cols_or_d2, int flags, float ignore_label, float alpha,
                                 void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  if (d0 == 0) {
    const int rows = rows_or_d1, cols = cols_or_d2;
    Tensor<gpu, 2, float> D = G2(dst, rows, cols, dstride, st.get());
    Tensor<gpu, 2, float> S = G2(src, rows, cols, sstride, st.get());
    Tensor<gpu, 1, float> L = G1(label, rows, st.get());
    switch (flags) {
      case 0: SoftmaxGrad(D, S, L); break;
      case 1: SmoothSoftmaxGrad(D, S, L, alpha); break;
      case 2: SoftmaxGrad(D, S, L, ignore_label); break;
      default: SmoothSoftmaxGrad(D, S, L, ignore_label, alpha); break;
    }
  } else {
    const int d1 = rows_or_d1, d2 = cols_or_d2;
    Tensor<gpu, 3, float> D = G3(dst, d0, d1, d2, dstride, st.get());
    Tensor<gpu, 3, float> S = G3(src, d0, d1, d2, sstride, st.get());
    Tensor<gpu, 2, float> L = G2(label, d0, d2, lstride, st.get());
    switch (flags) {
      case 0: SoftmaxGrad(D, S, L); break;
      case 1: SmoothSoftmaxGrad(D, S, L, alpha); break;
      case 2: SoftmaxGrad(D, S, L, ignore_label); break;
      default: SmoothSoftmaxGrad(D, S, L, ignore_label, alpha); break;
    }
  }
  CASE_END
}

int mshadow_case_softmax3d_f32(float *dst, int dstride, const float *src, int sstride, int d0,
                               int d1, int d2, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Softmax(G3(dst, d0, d1, d2, dstride, st.get()), G3(src, d0, d1, d2, sstride, st.get()));
  CASE_END
}

/* op: 0 AddTakeGrad(dst, index, src), 1 AddTakeGradLargeBatch(dst, sorted, index, src),
   2 IndexFill(dst, index, src); int32 index vectors */
int mshadow_case_rows_by_index_f32(int op, float *dst, int dstride, int k_rows, const int *sorted,
                                   const int *index, int n_index, const float *src, int sstride,
                                   int src_rows, int cols, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 2, float> D = G2(dst, k_rows, cols, dstride, st.get());
  Tensor<gpu, 2, float> S = G2(src, src_rows, cols, sstride, st.get());
  Tensor<gpu, 1, int> I(const_cast<int *>(index), Shape1(n_index), st.get());
  if (op == 0) {
    AddTakeGrad(D, I, S);
  } else if (op == 1) {
    Tensor<gpu, 1, int> Srt(const_cast<int *>(sorted), Shape1(n_index), st.get());
    AddTakeGradLargeBatch(D, Srt, I, S);
  } else {
    IndexFill(D, I, S);
  }
  CASE_END
}

/* the same families on tensors of another element type: type_flag 0 float, 1 double, 2 half_t
   (mshadow::TypeFlag codes). ignore_label is handed over as a double and converted to the
   element type, which is what a caller holding a DType would pass. */
int mshadow_case_grad_family_any(int type_flag, void *dst, int dstride, const void *src, int sstride,
                                 const void *label, int lstride, int d0, int rows_or_d1,
                                 int cols_or_d2, int flags, double ignore_label, float alpha,
                                 void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  MSHADOW_REAL_TYPE_SWITCH(type_flag, DType, {
    GradFamilyOf<DType>(dst, dstride, src, sstride, label, lstride, d0, rows_or_d1, cols_or_d2, flags,
                        ignore_label, alpha, st.get());
  });
  CASE_END
}

int mshadow_case_softmax3d_any(int type_flag, void *dst, int dstride, const void *src, int sstride,
                               int d0, int d1, int d2, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  MSHADOW_REAL_TYPE_SWITCH(type_flag, DType, {
    Softmax(G3(static_cast<const DType *>(dst), d0, d1, d2, dstride, st.get()),
            G3(static_cast<const DType *>(src), d0, d1, d2, sstride, st.get()));
  });
  CASE_END
}

/* op as for mshadow_case_rows_by_index_f32; index_flag: 0 float, 2 half_t, 4 int32, 6 int64 */
int mshadow_case_rows_by_index_any(int op, int type_flag, int index_flag, void *dst, int dstride,
                                   int k_rows, const void *sorted, const void *index, int n_index,
                                   const void *src, int sstride, int src_rows, int cols,
                                   void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  MSHADOW_REAL_TYPE_SWITCH(type_flag, DType, {
    RowsByIndexOfIndex<DType>(index_flag, op, dst, dstride, k_rows, sorted, index, n_index, src,
                              sstride, src_rows, cols, st.get());
  });
  CASE_END
}

/* index-remapping extensions through the generic expression kernel; dense tensors */
int mshadow_case_shaping_f32(int op, float *out, const float *a, const float *v, int n, int c,
                             int h, int w, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
#define OUT4(d0, d1, d2, d3) G4(out, d0, d1, d2, d3, d3, st.get())
#define OUT2(d0, d1) G2(out, d0, d1, d1, st.get())
#define IN4(d0, d1, d2, d3) G4(a, d0, d1, d2, d3, d3, st.get())
#define IN2(d0, d1) G2(a, d0, d1, d1, st.get())
#define VEC(len) G1(v, len, st.get())
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
  CASE_END
}

/* Random<gpu>: op 0 SampleUniform(p0, p1) into the first half and then into the second half of
   out; 1 SampleGaussian(p0, p1); 2 out = rnd.uniform(Shape1(n)) * 2; 3 GetRandInt (out holds
   unsigned words) */
int mshadow_case_random_f32(int op, int seed, float *out, int n, float p0, float p1, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Random<gpu, float> rnd(seed);
  rnd.set_stream(st.get());
  Tensor<gpu, 1, float> dst = G1(out, n, st.get());
  if (op == 0) {
    Tensor<gpu, 1, float> lo = dst.Slice(0, n / 2), hi = dst.Slice(n / 2, n);
    rnd.SampleUniform(&lo, p0, p1);
    rnd.SampleUniform(&hi, p0, p1);
  } else if (op == 1) {
    rnd.SampleGaussian(&dst, p0, p1);
  } else if (op == 2) {
    dst = rnd.uniform(Shape1(n)) * 2.0f;
  } else {
    rnd.GetRandInt(G1(reinterpret_cast<unsigned *>(out), n, st.get()));
  }
  st.get()->Wait();   // rnd's buffer is released when it goes out of scope
  CASE_END
}

/* the same through Random<gpu, double> (ops 0-2) */
int mshadow_case_random_f64(int op, int seed, double *out, int n, double p0, double p1, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Random<gpu, double> rnd(seed);
  rnd.set_stream(st.get());
  Tensor<gpu, 1, double> dst = G1(out, n, st.get());
  if (op == 0) {
    Tensor<gpu, 1, double> lo = dst.Slice(0, n / 2), hi = dst.Slice(n / 2, n);
    rnd.SampleUniform(&lo, p0, p1);
    rnd.SampleUniform(&hi, p0, p1);
  } else if (op == 1) {
    rnd.SampleGaussian(&dst, p0, p1);
  } else {
    dst = rnd.uniform(Shape1(n)) * 2.0;
  }
  st.get()->Wait();
  CASE_END
}

/* op 0: SortByKey(keys, values, is_ascend); op 1: VectorizedSort(keys as the values to sort,
   values as the segment numbers). key_kind 0: float keys / int values, 1: int keys / float
   values (for op 1 the segments are int either way) */
int mshadow_case_sort_by_key_32(int op, void *keys, int key_kind, void *values, int n,
                                int is_ascend, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  if (op == 0 && key_kind == 0) {
    SortByKey(G1(static_cast<float *>(keys), n, st.get()), G1(static_cast<int *>(values), n, st.get()),
              is_ascend != 0);
  } else if (op == 0) {
    SortByKey(G1(static_cast<int *>(keys), n, st.get()), G1(static_cast<float *>(values), n, st.get()),
              is_ascend != 0);
  } else if (key_kind == 0) {
    VectorizedSort(G1(static_cast<float *>(keys), n, st.get()),
                   G1(static_cast<int *>(values), n, st.get()));
  } else {
    VectorizedSort(G1(static_cast<int *>(keys), n, st.get()),
                   G1(static_cast<int *>(values), n, st.get()));
  }
  CASE_END
}

/* SortByKey(keys, values, is_ascend) for keys and values of any type of the type switch
   (mshadow::TypeFlag codes: 0 float, 1 double, 2 half_t, 3 uint8, 4 int32, 5 int8, 6 int64) */
int mshadow_case_sort_by_key_any(int key_flag, int value_flag, void *keys, void *values, int n,
                                 int is_ascend, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  MSHADOW_TYPE_SWITCH(key_flag, KDType, {
    MSHADOW_TYPE_SWITCH(value_flag, VDType, {
      SortByKey(G1(static_cast<KDType *>(keys), n, st.get()),
                G1(static_cast<VDType *>(values), n, st.get()), is_ascend != 0);
    });
  });
  CASE_END
}

/* caller-side functor of the extension cases (local response normalisation squares its input) */
struct square_of {
  MSHADOW_XINLINE static float Map(float a) { return a * a; }
};

/* channel pooling, axis reductions / broadcasts, permutations, assignable views and the
   index look-ups, through the generic expression kernel; dense tensors */
int mshadow_case_extensions_f32(int op, float *out, const float *a, const float *b, const float *c,
                                int n, int ch, int h, int w, int p0, int p1, int p2,
                                void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
#define TENSOR(dim) Tensor<gpu, dim, float>
#define V1(p, len) G1(p, len, st.get())
#define V2(p, d0, d1) G2(p, d0, d1, d1, st.get())
#define V3(p, d0, d1, d2) G3(p, d0, d1, d2, d2, st.get())
#define V4(p, d0, d1, d2, d3) G4(p, d0, d1, d2, d3, d3, st.get())
#define V4S(p, d0, d1, d2, d3, pitch) G4(p, d0, d1, d2, d3, pitch, st.get())
#include "./extension_cases.inc"
#undef TENSOR
#undef V1
#undef V2
#undef V3
#undef V4S
#undef V4
  CASE_END
}

/* matrix products through the expression engine, VectorDot and BatchGEMM; dense operands
   (shapes per op in dot_cases.inc) */
int mshadow_case_dot_f32(int op, float *out, const float *a, const float *b, int m, int k, int n,
                         int batch, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
#define XPU gpu
#define STREAM st.get()
#define TENSOR(dim) Tensor<gpu, dim, float>
#define V1(p, len) G1(p, len, st.get())
#define V2(p, d0, d1) G2(p, d0, d1, d1, st.get())
#define V2S(p, d0, d1, pitch) G2(p, d0, d1, pitch, st.get())
#define V3(p, d0, d1, d2) G3(p, d0, d1, d2, d2, st.get())
#include "./dot_cases.inc"
#undef XPU
#undef STREAM
#undef TENSOR
#undef V1
#undef V2
#undef V2S
#undef V3
  CASE_END
}

/* out = x * x + x over n pairs of binary16 values taken as half2_t elements */
int mshadow_case_half2_map(uint16_t *out, const uint16_t *x, int n_pairs, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  typedef half::half2_t H2;
  Tensor<gpu, 1, H2> X = G1(reinterpret_cast<const H2 *>(x), n_pairs, st.get());
  Tensor<gpu, 1, H2> O = G1(reinterpret_cast<const H2 *>(out), n_pairs, st.get());
  O = X * X + X;
  CASE_END
}

/* two_layer_net::Train on the device; every pointer is HOST memory (the program copies) */
int mshadow_case_two_layer_net_f32(int steps, float eta, float decay, int batch, int n_in,
                                   int n_hidden, int n_out, const float *x, const float *label,
                                   float *w1, float *w2, float *probs, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  two_layer_net::Train<gpu>(
      st.get(), steps, eta, decay,
      Tensor<cpu, 2, float>(const_cast<float *>(x), Shape2(batch, n_in)),
      Tensor<cpu, 1, float>(const_cast<float *>(label), Shape1(batch)),
      Tensor<cpu, 2, float>(w1, Shape2(n_in, n_hidden)),
      Tensor<cpu, 2, float>(w2, Shape2(n_hidden, n_out)),
      Tensor<cpu, 2, float>(probs, Shape2(batch, n_out)));
  CASE_END
}

/* conv_net::Train on the device; every pointer is HOST memory (the program copies) */
int mshadow_case_conv_net_f32(const int *geometry, int steps, float eta, float decay,
                              const float *images, const float *labels, const float *fixed_grad,
                              float *kernel, float *weight, float *const *keep, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  const conv_net::Geometry g = {geometry[0], geometry[1], geometry[2], geometry[3], geometry[4],
                                geometry[5], geometry[6], geometry[7], geometry[8]};
  conv_net::Train<gpu>(st.get(), g, steps, eta, decay, images, labels, fixed_grad, kernel, weight, keep);
  CASE_END
}

/* conv_net::ConvPair on the device for float (half == 0) or binary16 elements; HOST memory */
int mshadow_case_conv_pair(int half, const int *geometry, const void *image, const void *kernel,
                           const void *grad_out, void *col_forward, void *out, void *col_backward,
                           void *image_grad, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  const conv_net::Geometry g = {geometry[0], geometry[1], geometry[2], geometry[3], geometry[4],
                                geometry[5], geometry[6], geometry[7], geometry[8]};
  if (half) {
    conv_net::ConvPair<gpu, HalfT>(st.get(), g, static_cast<const HalfT *>(image),
                                   static_cast<const HalfT *>(kernel), static_cast<const HalfT *>(grad_out),
                                   static_cast<HalfT *>(col_forward), static_cast<HalfT *>(out),
                                   static_cast<HalfT *>(col_backward), static_cast<HalfT *>(image_grad));
  } else {
    conv_net::ConvPair<gpu, float>(st.get(), g, static_cast<const float *>(image),
                                   static_cast<const float *>(kernel), static_cast<const float *>(grad_out),
                                   static_cast<float *>(col_forward), static_cast<float *>(out),
                                   static_cast<float *>(col_backward), static_cast<float *>(image_grad));
  }
  CASE_END
}

int mshadow_case_pool_f32(float *dst, int dstride, const float *src, int sstride, int planes,
                          int h, int w, int ph, int pw, int ky, int kx, int sy, int sx,
                          int reducer, int variant, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 3, float> S = G3(src, planes, h, w, sstride, st.get());
  Tensor<gpu, 3, float> o = G3(dst, planes, ph, pw, dstride, st.get());
  const Shape<2> ps = Shape2(ph, pw);
  if (variant == 0) {
    if (reducer == 0) o = pool<red::sum>(S, ps, ky, kx, sy, sx);
    else if (reducer == 1) o = pool<red::maximum>(S, ps, ky, kx, sy, sx);
    else o = pool<red::minimum>(S, ps, ky, kx, sy, sx);
  } else {
    if (reducer == 0) o = pool<red::sum>(F<op::identity>(S), ps, ky, kx, sy, sx);
    else if (reducer == 1) o = pool<red::maximum>(F<op::identity>(S), ps, ky, kx, sy, sx);
    else o = pool<red::minimum>(F<op::identity>(S), ps, ky, kx, sy, sx);
  }
  CASE_END
}

int mshadow_case_unpool_f32(float *dst, int dstride, const float *src, int sstride,
                            const float *pooled, int pstride, const float *grad, int gstride,
                            int planes, int h, int w, int ph, int pw, int ky, int kx, int sy,
                            int sx, int reducer, int variant, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Tensor<gpu, 3, float> S = G3(src, planes, h, w, sstride, st.get());
  Tensor<gpu, 3, float> P = G3(pooled, planes, ph, pw, pstride, st.get());
  Tensor<gpu, 3, float> Gd = G3(grad, planes, ph, pw, gstride, st.get());
  Tensor<gpu, 3, float> o = G3(dst, planes, h, w, dstride, st.get());
  if (variant == 0) {
    if (reducer == 0) o = unpool<red::sum>(S, P, Gd, ky, kx, sy, sx);
    else if (reducer == 1) o = unpool<red::maximum>(S, P, Gd, ky, kx, sy, sx);
    else o = unpool<red::minimum>(S, P, Gd, ky, kx, sy, sx);
  } else {
    if (reducer == 0) {
      o = unpool<red::sum>(F<op::identity>(S), F<op::identity>(P), F<op::identity>(Gd), ky, kx, sy, sx);
    } else if (reducer == 1) {
      o = unpool<red::maximum>(F<op::identity>(S), F<op::identity>(P), F<op::identity>(Gd), ky, kx, sy, sx);
    } else {
      o = unpool<red::minimum>(F<op::identity>(S), F<op::identity>(P), F<op::identity>(Gd), ky, kx, sy, sx);
    }
  }
  CASE_END
}

#define CASE_IM2COL(NAME, CT, MT)                                                                \
  int NAME(CT *col, int cstride, const CT *img, int istride, int n, int c, int h, int w, int ky, \
           int kx, int sy, int sx, int dy, int dx, int pad_y, int pad_x, int variant,            \
           void *stream) {                                                                       \
    CASE_BEGIN                                                                                   \
    BorrowedStream st(stream);                                                                   \
    const int hp = h + 2 * pad_y, wp = w + 2 * pad_x;                                            \
    const int oh = (hp - (dy * (ky - 1) + 1)) / sy + 1, ow = (wp - (dx * (kx - 1) + 1)) / sx + 1; \
    Tensor<gpu, 4, MT> I = G4(reinterpret_cast<const MT *>(img), n, c, h, w, istride, st.get()); \
    Tensor<gpu, 2, MT> O =                                                                       \
        G2(reinterpret_cast<MT *>(col), ky * kx * c, oh * ow * n, cstride, st.get());            \
    if (variant == 0) O = unpack_patch2col(pad(I, pad_y, pad_x), ky, kx, sy, sx, dy, dx);        \
    else O = unpack_patch2col(pad(F<op::identity>(I), pad_y, pad_x), ky, kx, sy, sx, dy, dx);    \
    CASE_END                                                                                     \
  }
CASE_IM2COL(mshadow_case_im2col_f16, uint16_t, half::half_t)
CASE_IM2COL(mshadow_case_im2col_f32, float, float)

#define CASE_COL2IM(NAME, CT, MT)                                                                \
  int NAME(CT *img, int istride, const CT *col, int cstride, int n, int c, int h, int w, int ky, \
           int kx, int sy, int sx, int dy, int dx, int pad_y, int pad_x, int variant,            \
           void *stream) {                                                                       \
    CASE_BEGIN                                                                                   \
    BorrowedStream st(stream);                                                                   \
    const int hp = h + 2 * pad_y, wp = w + 2 * pad_x;                                            \
    const int oh = (hp - (dy * (ky - 1) + 1)) / sy + 1, ow = (wp - (dx * (kx - 1) + 1)) / sx + 1; \
    Tensor<gpu, 4, MT> I = G4(reinterpret_cast<MT *>(img), n, c, h, w, istride, st.get());       \
    Tensor<gpu, 2, MT> C =                                                                       \
        G2(reinterpret_cast<const MT *>(col), ky * kx * c, oh * ow * n, cstride, st.get());      \
    if (variant == 0) {                                                                          \
      I = crop(pack_col2patch(C, Shape4(n, c, hp, wp), ky, kx, sy, sx, dy, dx), Shape2(h, w),    \
               pad_y, pad_x);                                                                    \
    } else {                                                                                     \
      I = crop(pack_col2patch(F<op::identity>(C), Shape4(n, c, hp, wp), ky, kx, sy, sx, dy, dx), \
               Shape2(h, w), pad_y, pad_x);                                                      \
    }                                                                                            \
    CASE_END                                                                                     \
  }
CASE_COL2IM(mshadow_case_col2im_f16, uint16_t, half::half_t)
CASE_COL2IM(mshadow_case_col2im_f32, float, float)

int mshadow_case_copy_d2d_f32(float *dst, int dstride, const float *src, int sstride, int rows,
                              int cols, void *stream) {
  CASE_BEGIN
  BorrowedStream st(stream);
  Copy(G2(dst, rows, cols, dstride, st.get()), G2(src, rows, cols, sstride, st.get()), st.get());
  CASE_END
}

int mshadow_case_copy_roundtrip_f32(float *host_out, const float *host_in, int rows, int cols,
                                    int pad, int *device_stride) {
  CASE_BEGIN
  InitTensorEngine<gpu>(0);
  Stream<gpu> *stream = NewStream<gpu>(0);
  {
    Tensor<cpu, 2, float> hin(const_cast<float *>(host_in), Shape2(rows, cols));
    Tensor<cpu, 2, float> hout(host_out, Shape2(rows, cols));
    TensorContainer<gpu, 2, float> a(pad != 0), b(pad != 0);
    a.set_stream(stream);
    b.set_stream(stream);
    a.Resize(Shape2(rows, cols));
    b.Resize(Shape2(rows, cols));
    if (device_stride != NULL) *device_stride = a.stride_;
    Copy(a, hin, stream);
    Copy(b, a, stream);
    b += 0.0f;  // an expression on a possibly pitched container
    Copy(hout, b, stream);
    stream->Wait();
  }
  DeleteStream(stream);
  ShutdownTensorEngine<gpu>();
  CASE_END
}

}  // extern "C"
