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

template <int dim, typename DType>
inline void Copy(Tensor<cpu, dim, DType> _dst, const Tensor<cpu, dim, DType> &_src,
                 Stream<cpu> *stream) {
  CHECK_EQ(_dst.shape_, _src.shape_)
      << "Copy:shape mismatch:" << _dst.shape_ << " vs " << _src.shape_;
  if (_dst.CheckContiguous() && _src.CheckContiguous()) {
    memcpy(_dst.dptr_, _src.dptr_, sizeof(DType) * _dst.shape_.Size());
    return;
  }
  Tensor<cpu, 2, DType> dst = _dst.FlatTo2D();
  Tensor<cpu, 2, DType> src = _src.FlatTo2D();
  for (index_t y = 0; y < dst.size(0); ++y) {
    memcpy(dst[y].dptr_, src[y].dptr_, sizeof(DType) * dst.size(1));
  }
}

/*! \brief the host evaluation loop: rows in parallel, columns in order */
template <typename Saver, typename R, int dim, typename DType, typename E>
inline void MapPlan(TRValue<R, cpu, dim, DType> *dst, const expr::Plan<E, DType> &plan) {
  Shape<2> shape = expr::ShapeCheck<dim, R>::Check(dst->self()).FlatTo2D();
  expr::Plan<R, DType> dplan = expr::MakePlan(dst->self());
#pragma omp parallel for
  for (openmp_index_t y = 0; y < shape[0]; ++y) {
    for (index_t x = 0; x < shape[1]; ++x) {
      Saver::template Save<DType>(dplan.REval(y, x), plan.Eval(y, x));
    }
  }
}

template <typename Saver, typename R, int dim, typename DType, typename E, int etype>
inline void MapExp(TRValue<R, cpu, dim, DType> *dst, const expr::Exp<E, DType, etype> &exp) {
  expr::TypeCheckPass<expr::TypeCheck<cpu, dim, DType, E>::kMapPass>::
      Error_All_Tensor_in_Exp_Must_Have_Same_Type();
  Shape<dim> eshape = expr::ShapeCheck<dim, E>::Check(exp.self());
  Shape<dim> dshape = expr::ShapeCheck<dim, R>::Check(dst->self());
  CHECK(eshape[0] == 0 || eshape == dshape)
      << "Assignment: Shape of Tensors are not consistent with target, "
      << "eshape: " << eshape << " dshape:" << dshape;
  MapPlan<Saver>(dst, expr::MakePlan(exp.self()));
}

template <typename Saver, typename Reducer, typename R, typename DType, typename E, int etype>
inline void MapReduceKeepLowest(TRValue<R, cpu, 1, DType> *dst,
                                const expr::Exp<E, DType, etype> &exp, DType scale) {
  expr::TypeCheckPass<expr::TypeCheck<cpu, 1, DType, E>::kRedPass>::
      Error_TypeCheck_Not_Pass_For_Reduce_Exp();
  Shape<2> eshape = expr::ShapeCheck<expr::ExpInfo<E>::kDim, E>::Check(exp.self()).FlatTo2D();
  Shape<1> dshape = expr::ShapeCheck<1, R>::Check(dst->self());
  CHECK_EQ(eshape[1], dshape[0]) << "MapReduceKeepLowest::reduction dimension do not match";
  CHECK_NE(eshape[0], 0U) << "can not reduce over empty tensor";
  expr::Plan<R, DType> dplan = expr::MakePlan(dst->self());
  expr::Plan<E, DType> splan = expr::MakePlan(exp.self());
#pragma omp parallel for
  for (openmp_index_t x = 0; x < eshape[1]; ++x) {
    DType res = splan.Eval(0, x);
    for (index_t y = 1; y < eshape[0]; ++y) Reducer::Reduce(res, splan.Eval(y, x));
    Saver::template Save<DType>(dplan.REval(0, x), res * scale);
  }
}

template <typename Saver, typename Reducer, int dimkeep, typename R, typename DType, typename E,
          int etype>
inline void MapReduceKeepHighDim(TRValue<R, cpu, 1, DType> *dst,
                                 const expr::Exp<E, DType, etype> &exp, DType scale) {
  expr::TypeCheckPass<expr::TypeCheck<cpu, dimkeep, DType, E>::kRedPass>::
      Error_TypeCheck_Not_Pass_For_Reduce_Exp();
  typedef Shape<expr::ExpInfo<E>::kDim> EShape;
  EShape eshape = expr::ShapeCheck<expr::ExpInfo<E>::kDim, E>::Check(exp.self());
  Shape<1> dshape = expr::ShapeCheck<1, R>::Check(dst->self());
  CHECK_EQ(eshape[dimkeep], dshape[0]) << "MapReduceKeepHighDim::reduction dimension do not match";
  /* (outer, kept, inner rows, last dim) */
  const index_t n_out = eshape.ProdShape(0, dimkeep);
  const index_t n_keep = eshape[dimkeep];
  const index_t n_y = eshape.ProdShape(dimkeep + 1, EShape::kSubdim);
  const index_t n_x = eshape[EShape::kSubdim];
  expr::Plan<R, DType> dplan = expr::MakePlan(dst->self());
  expr::Plan<E, DType> splan = expr::MakePlan(exp.self());
#pragma omp parallel for
  for (openmp_index_t c = 0; c < n_keep; ++c) {
    DType res;
    Reducer::SetInitValue(res);
    for (index_t n = 0; n < n_out; ++n) {
      DType tres;
      Reducer::SetInitValue(tres);
      for (index_t y = 0; y < n_y; ++y) {
        for (index_t x = 0; x < n_x; ++x) {
          Reducer::Reduce(tres, splan.Eval((n * n_keep + c) * n_y + y, x));
        }
      }
      Reducer::Reduce(res, tres);
    }
    Saver::template Save<DType>(dplan.REval(0, c), DType(res * scale));
  }
}

/*! \brief one row: max, exp(x - max) summed left to right, then divide */
template <typename DType>
inline void Softmax(Tensor<cpu, 1, DType> dst, const Tensor<cpu, 1, DType> &energy) {
  DType mmax = energy[0];
  for (index_t x = 1; x < dst.size(0); ++x) {
    if (mmax < energy[x]) mmax = energy[x];
  }
  DType sum = DType(0.0f);
  for (index_t x = 0; x < dst.size(0); ++x) {
    dst[x] = std::exp(energy[x] - mmax);
    sum += dst[x];
  }
  for (index_t x = 0; x < dst.size(0); ++x) dst[x] /= sum;
}
template <typename DType>
inline void Softmax(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &energy) {
  CHECK_EQ(dst.shape_, energy.shape_) << "Softmax: shape mismatch";
#pragma omp parallel for
  for (openmp_index_t y = 0; y < dst.size(0); ++y) Softmax(dst[y], energy[y]);
}
template <typename DType>
inline void SoftmaxGrad(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &src,
                        const Tensor<cpu, 1, DType> &label) {
#pragma omp parallel for
  for (openmp_index_t y = 0; y < dst.size(0); ++y) {
    const index_t k = static_cast<int>(label[y]);
    for (index_t x = 0; x < dst.size(1); ++x) {
      if (x == k) {
        dst[y][k] = src[y][k] - 1.0f;
      } else {
        dst[y][x] = src[y][x];
      }
    }
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
/*! \brief softmax over the middle dimension of (d0, d1, d2) */
template <typename DType>
inline void Softmax(Tensor<cpu, 3, DType> dst, const Tensor<cpu, 3, DType> &energy) {
  CHECK_EQ(dst.shape_, energy.shape_) << "Softmax: shape mismatch";
#pragma omp parallel for
  for (openmp_index_t y = 0; y < dst.size(0); ++y) {
    for (index_t n = 0; n < dst.size(2); ++n) {
      DType mmax = energy[y][0][n];
      for (index_t x = 1; x < dst.size(1); ++x) {
        if (mmax < energy[y][x][n]) mmax = energy[y][x][n];
      }
      DType sum = DType(0.0f);
      for (index_t x = 0; x < dst.size(1); ++x) {
        dst[y][x][n] = std::exp(energy[y][x][n] - mmax);
        sum += dst[y][x][n];
      }
      for (index_t x = 0; x < dst.size(1); ++x) dst[y][x][n] /= sum;
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
