/*
 * Tensor<cpu>: host-side device of the API (staging buffers, small host tensors,
 * code templated on the device tag). Loop orders restate
 * mshadow/tensor_cpu-inl.h:97-302 and :464-472 of the reference so that a program
 * run with xpu = cpu produces the reference's values. Nothing here is used by, or
 * substituted for, any Tensor<gpu> operation.
 */
#ifndef MSHADOW_CPU_TENSOR_CPU_H_
#define MSHADOW_CPU_TENSOR_CPU_H_

#include <algorithm>
#include <vector>
#include <cmath>
#include <cstdlib>
#include <cstring>

#include "../tensor.h"

namespace mshadow {

template <>
inline void InitTensorEngine<cpu>(int dev_id) {}
template <>
inline void ShutdownTensorEngine<cpu>(void) {}
template <>
inline void SetDevice<cpu>(int devid) {}
template <>
inline Stream<cpu> *NewStream<cpu>(bool create_blas_handle, bool create_dnn_handle, int dev_id) {
  return new Stream<cpu>();
}
template <>
inline void DeleteStream<cpu>(Stream<cpu> *stream) {
  delete stream;
}

namespace cpu_detail {
/*! \brief rows of `width_bytes`, each starting on a 16-byte boundary
 *  (mshadow/packet-inl.h:59-78: pitch = width rounded up to 16 bytes) */
inline void *AllocPitch(size_t *pitch_bytes, size_t width_bytes, size_t rows) {
  const size_t unit = 16;
  const size_t pitch = (width_bytes + unit - 1) / unit * unit;
  *pitch_bytes = pitch;
  void *p = NULL;
  const size_t total = pitch * rows;
  int ret = posix_memalign(&p, unit, total ? total : unit);
  CHECK_EQ(ret, 0) << "AlignedMallocPitch failed";
  return p;
}
}  // namespace cpu_detail

template <typename xpu>
inline void *AllocHost_(size_t size);
template <typename xpu>
inline void FreeHost_(void *dptr);
template <>
inline void *AllocHost_<cpu>(size_t size) {
  size_t pitch;
  return cpu_detail::AllocPitch(&pitch, size, 1);
}
template <>
inline void FreeHost_<cpu>(void *dptr) {
  free(dptr);
}
/*! \brief host tensor whose memory suits transfers to xpu (pinned for gpu) */
template <typename xpu, int dim, typename DType>
inline void AllocHost(Tensor<cpu, dim, DType> *obj) {
  obj->stride_ = obj->size(dim - 1);
  CHECK_EQ(obj->CheckContiguous(), true) << "AllocHost";
  void *dptr = AllocHost_<xpu>(obj->MSize() * sizeof(DType));
  obj->dptr_ = reinterpret_cast<DType *>(dptr);
}
template <typename xpu, int dim, typename DType>
inline void FreeHost(Tensor<cpu, dim, DType> *obj) {
  if (obj->dptr_ == NULL) {
    LOG(FATAL) << "FreeHost:: double free";
  }
  FreeHost_<xpu>(obj->dptr_);
  obj->dptr_ = NULL;
}

template <int dim, typename DType>
inline void AllocSpace(Tensor<cpu, dim, DType> *obj, bool pad) {
  size_t pitch;
  void *dptr;
  if (pad) {
    dptr = cpu_detail::AllocPitch(&pitch, obj->size(dim - 1) * sizeof(DType),
                                  obj->shape_.FlatTo2D()[0]);
    obj->stride_ = static_cast<index_t>(pitch / sizeof(DType));
  } else {
    obj->stride_ = obj->size(dim - 1);
    dptr = cpu_detail::AllocPitch(&pitch, obj->shape_.Size() * sizeof(DType), 1);
  }
  obj->dptr_ = reinterpret_cast<DType *>(dptr);
}
template <int dim, typename DType>
inline void FreeSpace(Tensor<cpu, dim, DType> *obj) {
  free(obj->dptr_);
  obj->dptr_ = NULL;
}
template <typename Device, typename DType, int dim>
inline Tensor<Device, dim, DType> NewTensor(const Shape<dim> &shape, DType initv, bool pad,
                                            Stream<Device> *stream_) {
  Tensor<Device, dim, DType> obj(shape);
  obj.stream_ = stream_;
  AllocSpace(&obj, pad);
  MapExp<sv::saveto>(&obj, expr::ScalarExp<DType>(initv));
  return obj;
}

/*! \brief element-for-element copy between two host tensors of one shape (either may be
 *  pitched): one block when both are dense, otherwise row by row */
template <int dim, typename DType>
inline void Copy(Tensor<cpu, dim, DType> to, const Tensor<cpu, dim, DType> &from,
                 Stream<cpu> *stream) {
  CHECK_EQ(to.shape_, from.shape_) << "Copy:shape mismatch:" << to.shape_ << " vs " << from.shape_;
  const Shape<2> flat = to.shape_.FlatTo2D();
  const size_t row_bytes = sizeof(DType) * flat[1];
  if (to.stride_ == flat[1] && from.stride_ == flat[1]) {
    memcpy(to.dptr_, from.dptr_, row_bytes * flat[0]);
    return;
  }
  for (index_t r = 0; r < flat[0]; ++r) {
    memcpy(to.dptr_ + static_cast<size_t>(r) * to.stride_,
           from.dptr_ + static_cast<size_t>(r) * from.stride_, row_bytes);
  }
}

namespace cpu_detail {
/*! \brief destination and source plans of one assignment or reduction, with the checked
 *  (rows, columns) extent of the source */
template <typename R, typename E, typename DType>
struct PlanPair {
  expr::Plan<R, DType> out;
  expr::Plan<E, DType> in;
  PlanPair(const R &dst, const E &src) : out(expr::MakePlan(dst)), in(expr::MakePlan(src)) {}
};
}  // namespace cpu_detail

/*! \brief the host evaluation loop: rows in parallel, columns in order */
template <typename Saver, typename R, int dim, typename DType, typename E>
inline void MapPlan(TRValue<R, cpu, dim, DType> *dst, const expr::Plan<E, DType> &plan) {
  const Shape<2> extent = expr::ShapeCheck<dim, R>::Check(dst->self()).FlatTo2D();
  expr::Plan<R, DType> target = expr::MakePlan(dst->self());
  const openmp_index_t rows = extent[0];
  const index_t cols = extent[1];
#pragma omp parallel for
  for (openmp_index_t r = 0; r < rows; ++r) {
    for (index_t c = 0; c < cols; ++c) Saver::template Save<DType>(target.REval(r, c), plan.Eval(r, c));
  }
}

template <typename Saver, typename R, int dim, typename DType, typename E, int etype>
inline void MapExp(TRValue<R, cpu, dim, DType> *dst, const expr::Exp<E, DType, etype> &exp) {
  expr::TypeCheckPass<expr::TypeCheck<cpu, dim, DType, E>::kMapPass>::
      Error_All_Tensor_in_Exp_Must_Have_Same_Type();
  const Shape<dim> want = expr::ShapeCheck<dim, R>::Check(dst->self());
  const Shape<dim> have = expr::ShapeCheck<dim, E>::Check(exp.self());
  /* a shape whose first extent is 0 is a scalar-like expression that fits any target */
  CHECK(have[0] == 0 || have == want)
      << "Assignment: Shape of Tensors are not consistent with target, "
      << "eshape: " << have << " dshape:" << want;
  MapPlan<Saver>(dst, expr::MakePlan(exp.self()));
}

/*! \brief dst[x] <saver>= scale * reduce over y of exp(y, x): every column is one serial chain
 *  that starts from the element of row 0 (not from the reducer's initial value) and takes
 *  the rows in order; columns run in parallel */
template <typename Saver, typename Reducer, typename R, typename DType, typename E, int etype>
inline void MapReduceKeepLowest(TRValue<R, cpu, 1, DType> *dst,
                                const expr::Exp<E, DType, etype> &exp, DType scale) {
  expr::TypeCheckPass<expr::TypeCheck<cpu, 1, DType, E>::kRedPass>::
      Error_TypeCheck_Not_Pass_For_Reduce_Exp();
  const Shape<2> extent = expr::ShapeCheck<expr::ExpInfo<E>::kDim, E>::Check(exp.self()).FlatTo2D();
  const Shape<1> target = expr::ShapeCheck<1, R>::Check(dst->self());
  CHECK_EQ(extent[1], target[0]) << "MapReduceKeepLowest::reduction dimension do not match";
  CHECK_NE(extent[0], 0U) << "can not reduce over empty tensor";
  cpu_detail::PlanPair<R, E, DType> plans(dst->self(), exp.self());
  const openmp_index_t cols = extent[1];
  const index_t rows = extent[0];
#pragma omp parallel for
  for (openmp_index_t c = 0; c < cols; ++c) {
    DType acc = plans.in.Eval(0, c);
    for (index_t r = 1; r < rows; ++r) Reducer::Reduce(acc, plans.in.Eval(r, c));
    Saver::template Save<DType>(plans.out.REval(0, c), acc * scale);
  }
}

/*! \brief dst[c] <saver>= scale * reduce of exp over every axis but `dimkeep`. The source is
 *  viewed as (before, kept, rows behind, last axis); for a kept index the elements behind each
 *  `before` index are reduced first, in memory order, into a partial result that starts from
 *  the reducer's initial value, and the partial results are then reduced in `before` order -
 *  two levels, which a floating-point sum can tell from one */
template <typename Saver, typename Reducer, int dimkeep, typename R, typename DType, typename E,
          int etype>
inline void MapReduceKeepHighDim(TRValue<R, cpu, 1, DType> *dst,
                                 const expr::Exp<E, DType, etype> &exp, DType scale) {
  expr::TypeCheckPass<expr::TypeCheck<cpu, dimkeep, DType, E>::kRedPass>::
      Error_TypeCheck_Not_Pass_For_Reduce_Exp();
  typedef Shape<expr::ExpInfo<E>::kDim> SourceShape;
  const SourceShape extent = expr::ShapeCheck<expr::ExpInfo<E>::kDim, E>::Check(exp.self());
  const Shape<1> target = expr::ShapeCheck<1, R>::Check(dst->self());
  CHECK_EQ(extent[dimkeep], target[0]) << "MapReduceKeepHighDim::reduction dimension do not match";
  const index_t before = extent.ProdShape(0, dimkeep);
  const openmp_index_t kept = extent[dimkeep];
  const index_t rows_behind = extent.ProdShape(dimkeep + 1, SourceShape::kSubdim);
  const index_t last = extent[SourceShape::kSubdim];
  cpu_detail::PlanPair<R, E, DType> plans(dst->self(), exp.self());
#pragma omp parallel for
  for (openmp_index_t c = 0; c < kept; ++c) {
    DType total;
    Reducer::SetInitValue(total);
    for (index_t b = 0; b < before; ++b) {
      DType partial;
      Reducer::SetInitValue(partial);
      const index_t first_row = (b * static_cast<index_t>(kept) + static_cast<index_t>(c)) * rows_behind;
      for (index_t r = first_row; r < first_row + rows_behind; ++r) {
        for (index_t x = 0; x < last; ++x) Reducer::Reduce(partial, plans.in.Eval(r, x));
      }
      Reducer::Reduce(total, partial);
    }
    Saver::template Save<DType>(plans.out.REval(0, c), DType(total * scale));
  }
}

namespace cpu_detail {
/*! \brief softmax of `count` elements `step` apart, in the element type's own arithmetic:
 *  the largest element by strict <, exp(x - largest) stored and summed left to right, every
 *  stored term divided by the sum. The 1-D, 2-D and 3-D functions are this on different
 *  strides (mshadow/tensor_cpu-inl.h:270-285, 466-488). */
template <typename DType>
inline void SoftmaxStrided(DType *out, size_t out_step, const DType *in, size_t in_step,
                           index_t count) {
  DType largest = in[0];
  for (index_t i = 1; i < count; ++i) {
    if (largest < in[i * in_step]) largest = in[i * in_step];
  }
  DType denominator = DType(0.0f);
  for (index_t i = 0; i < count; ++i) {
    out[i * out_step] = std::exp(in[i * in_step] - largest);
    denominator += out[i * out_step];
  }
  for (index_t i = 0; i < count; ++i) out[i * out_step] /= denominator;
}
}  // namespace cpu_detail

template <typename DType>
inline void Softmax(Tensor<cpu, 1, DType> dst, const Tensor<cpu, 1, DType> &energy) {
  cpu_detail::SoftmaxStrided(dst.dptr_, 1, energy.dptr_, 1, dst.size(0));
}
template <typename DType>
inline void Softmax(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &energy) {
  CHECK_EQ(dst.shape_, energy.shape_) << "Softmax: shape mismatch";
  const openmp_index_t rows = dst.size(0);
#pragma omp parallel for
  for (openmp_index_t r = 0; r < rows; ++r) {
    cpu_detail::SoftmaxStrided(dst.dptr_ + static_cast<size_t>(r) * dst.stride_, 1,
                               energy.dptr_ + static_cast<size_t>(r) * energy.stride_, 1, dst.size(1));
  }
}

/* ---- the rest of the softmax family and the row scatter / gather functions
 * (mshadow/tensor_cpu-inl.h:304-528 of the reference). One element of every gradient
 * variant is GradValue(): smooth spreads alpha over the other classes, a row whose label
 * equals ignore_label gets zeros. */
namespace cpu_detail {
template <typename DType>
inline DType GradValue(DType s, bool at_label, bool smooth, float alpha, float smooth_grad) {
  if (at_label) return smooth ? DType(s - 1.0f + alpha) : DType(s - 1.0f);
  return smooth ? DType(s - smooth_grad) : s;
}
template <typename DType>
inline void Grad2D(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &src,
                   const Tensor<cpu, 1, DType> &label, bool use_ignore, int ignore, bool smooth,
                   float alpha) {
  const float smooth_grad = alpha / (dst.size(1) - 1);
#pragma omp parallel for
  for (openmp_index_t y = 0; y < dst.size(0); ++y) {
    const int k = static_cast<int>(label[y]);
    for (int x = 0; x < static_cast<int>(dst.size(1)); ++x) {
      dst[y][x] = (use_ignore && ignore == k) ? DType(0.0f)
                                              : GradValue(src[y][x], x == k, smooth, alpha, smooth_grad);
    }
  }
}
template <typename DType>
inline void Grad3D(Tensor<cpu, 3, DType> dst, const Tensor<cpu, 3, DType> &src,
                   const Tensor<cpu, 2, DType> &label, bool use_ignore, int ignore, bool smooth,
                   float alpha) {
  const float smooth_grad = alpha / (dst.size(1) - 1);
#pragma omp parallel for
  for (openmp_index_t n = 0; n < dst.size(2); ++n) {
    for (index_t y = 0; y < dst.size(0); ++y) {
      const int k = static_cast<int>(label[y][n]);
      for (int x = 0; x < static_cast<int>(dst.size(1)); ++x) {
        dst[y][x][n] = (use_ignore && ignore == k)
                           ? DType(0.0f)
                           : GradValue(src[y][x][n], x == k, smooth, alpha, smooth_grad);
      }
    }
  }
}
}  // namespace cpu_detail

template <typename DType>
inline void SoftmaxGrad(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &src,
                        const Tensor<cpu, 1, DType> &label) {
  cpu_detail::Grad2D(dst, src, label, false, 0, false, 0.0f);
}
template <typename DType>
inline void SmoothSoftmaxGrad(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &src,
                              const Tensor<cpu, 1, DType> &label, const float alpha) {
  cpu_detail::Grad2D(dst, src, label, false, 0, true, alpha);
}
template <typename DType>
inline void SoftmaxGrad(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &src,
                        const Tensor<cpu, 1, DType> &label, const DType &ignore_label) {
  cpu_detail::Grad2D(dst, src, label, true, static_cast<int>(ignore_label), false, 0.0f);
}
template <typename DType>
inline void SmoothSoftmaxGrad(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &src,
                              const Tensor<cpu, 1, DType> &label, const DType &ignore_label,
                              const float alpha) {
  cpu_detail::Grad2D(dst, src, label, true, static_cast<int>(ignore_label), true, alpha);
}
template <typename DType>
inline void SoftmaxGrad(Tensor<cpu, 3, DType> dst, const Tensor<cpu, 3, DType> &src,
                        const Tensor<cpu, 2, DType> &label) {
  cpu_detail::Grad3D(dst, src, label, false, 0, false, 0.0f);
}
template <typename DType>
inline void SmoothSoftmaxGrad(Tensor<cpu, 3, DType> dst, const Tensor<cpu, 3, DType> &src,
                              const Tensor<cpu, 2, DType> &label, const float alpha) {
  cpu_detail::Grad3D(dst, src, label, false, 0, true, alpha);
}
template <typename DType>
inline void SoftmaxGrad(Tensor<cpu, 3, DType> dst, const Tensor<cpu, 3, DType> &src,
                        const Tensor<cpu, 2, DType> &label, const DType &ignore_label) {
  cpu_detail::Grad3D(dst, src, label, true, static_cast<int>(ignore_label), false, 0.0f);
}
template <typename DType>
inline void SmoothSoftmaxGrad(Tensor<cpu, 3, DType> dst, const Tensor<cpu, 3, DType> &src,
                              const Tensor<cpu, 2, DType> &label, const DType &ignore_label,
                              const float alpha) {
  cpu_detail::Grad3D(dst, src, label, true, static_cast<int>(ignore_label), true, alpha);
}
/*! \brief softmax over the middle dimension of (d0, d1, d2): element (y, x, n) is
 *  (y * d1 + x) * stride + n, so a column (y, n) is d1 elements one pitch apart */
template <typename DType>
inline void Softmax(Tensor<cpu, 3, DType> dst, const Tensor<cpu, 3, DType> &energy) {
  CHECK_EQ(dst.shape_, energy.shape_) << "Softmax: shape mismatch";
  const openmp_index_t outer = dst.size(0);
  const index_t classes = dst.size(1), inner = dst.size(2);
#pragma omp parallel for
  for (openmp_index_t y = 0; y < outer; ++y) {
    DType *out = dst.dptr_ + static_cast<size_t>(y) * classes * dst.stride_;
    const DType *in = energy.dptr_ + static_cast<size_t>(y) * classes * energy.stride_;
    for (index_t n = 0; n < inner; ++n) {
      cpu_detail::SoftmaxStrided(out + n, dst.stride_, in + n, energy.stride_, classes);
    }
  }
}
/*! \brief dst[clamp(index[y])] += src[y], front to back */
template <typename IndexType, typename DType>
inline void AddTakeGrad(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 1, IndexType> &index,
                        const Tensor<cpu, 2, DType> &src) {
  const int K = dst.shape_[0];
  for (index_t y = 0; y < index.size(0); ++y) {
    int j = index[y];
    j = j <= 0 ? 0 : (j >= K ? K - 1 : j);
    dst[j] += src[y];
  }
}
/*! \brief dst[sorted[y]] += src[index[y]], front to back */
template <typename IndexType, typename DType>
inline void AddTakeGradLargeBatch(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 1, IndexType> &sorted,
                                  const Tensor<cpu, 1, IndexType> &index,
                                  const Tensor<cpu, 2, DType> &src) {
  for (index_t y = 0; y < sorted.size(0); ++y) dst[sorted[y]] += src[index[y]];
}
/*! \brief dst[index[y]] = src[y], front to back */
template <typename IndexType, typename DType>
inline void IndexFill(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 1, IndexType> &index,
                      const Tensor<cpu, 2, DType> &src) {
  for (index_t y = 0; y < index.size(0); ++y) {
    for (index_t j = 0; j < src.size(1); j++) dst[index[y]][j] = src[y][j];
  }
}

/*! \brief mshadow/tensor_cpu-inl.h:531-559 of the reference: positions are sorted stably
 *  under keys[i1] < keys[i2] (ascending) or > (descending), then both vectors are
 *  permuted */
template <typename KDType, typename VDType>
inline void SortByKey(Tensor<cpu, 1, KDType> keys, Tensor<cpu, 1, VDType> values,
                      bool is_ascend) {
  CHECK_EQ(keys.CheckContiguous(), true);
  CHECK_EQ(values.CheckContiguous(), true);
  CHECK_EQ(keys.size(0), values.size(0))
      << "The sizes of key/value are not equal! keys_size: " << keys.size(0)
      << "values_size: " << values.size(0);
  const index_t n = keys.size(0);
  std::vector<KDType> k(keys.dptr_, keys.dptr_ + n);
  std::vector<VDType> v(values.dptr_, values.dptr_ + n);
  std::vector<index_t> order(n);
  for (index_t i = 0; i < n; ++i) order[i] = i;
  if (is_ascend) {
    std::stable_sort(order.begin(), order.end(),
                     [&k](index_t a, index_t b) { return k[a] < k[b]; });
  } else {
    std::stable_sort(order.begin(), order.end(),
                     [&k](index_t a, index_t b) { return k[a] > k[b]; });
  }
  for (index_t i = 0; i < n; ++i) {
    keys[i] = k[order[i]];
    values[i] = v[order[i]];
  }
}
/*! \brief two stable sorts: by value, then by segment number (tensor_cpu-inl.h:561-566) */
template <typename Device, typename VDType, typename SDType>
inline void VectorizedSort(Tensor<Device, 1, VDType> values, Tensor<Device, 1, SDType> segments) {
  SortByKey(values, segments, true);
  SortByKey(segments, values, true);
}

}  // namespace mshadow
#endif  // MSHADOW_CPU_TENSOR_CPU_H_
