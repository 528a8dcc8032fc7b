/*
 * mshadow for gfx950: the one header callers include.
 *
 *   #include <mshadow/tensor.h>
 *   Tensor<gpu, 2> dst = ..., a = ..., b = ...;
 *   dst = a * b + 0.5f * F<sigmoid>(c) - d;     // one HIP kernel, 128-bit accesses
 *   v   = sumall_except_dim<1>(x4d);            // order-faithful wave64 reduction
 *   Softmax(p, logits);
 *
 * Declarations of the device functions follow mshadow/tensor.h:616-1050 of the
 * reference (names, template parameter order, default arguments). Definitions:
 * cpu/tensor_cpu.h for Tensor<cpu>, hip/tensor_gpu.h for Tensor<gpu>. A translation
 * unit compiled by a host compiler gets memory, copy, stream and the fixed-function
 * operations for Tensor<gpu> (they live behind the C ABI of libmshadow_hip);
 * evaluating arbitrary expressions into a Tensor<gpu> needs hipcc, because the
 * kernel is instantiated from the caller's expression type.
 */
#ifndef MSHADOW_TENSOR_H_
#define MSHADOW_TENSOR_H_

#include <iostream>
#include <string>

#include "./base.h"
#include "./core/tensor_types.h"
#include "./expr/traits.h"
#include "./expression.h"

namespace mshadow {

/*! \brief select and initialise a device; needed before any GPU tensor operation */
template <typename Device>
inline void InitTensorEngine(int device_id = 0);
/*! \brief counterpart of InitTensorEngine */
template <typename Device>
inline void ShutdownTensorEngine(void);
/*! \brief make devid the calling thread's current device */
template <typename Device>
inline void SetDevice(int devid);
/*! \brief create a computation stream; the two flags ask for BLAS / DNN handles, which
 *  callers do not hold here (they are accepted and ignored) */
template <typename Device>
inline Stream<Device> *NewStream(bool create_blas_handle, bool create_dnn_handle, int dev_id = -1);
/*! \brief the default of dev_id is an addition: guide/basic_stream.cu of the reference calls
 *  NewStream<gpu>() with no argument, which its own header (tensor.h:658-661) does not accept */
template <typename Device>
inline Stream<Device> *NewStream(int dev_id = -1) {
  return NewStream<Device>(true, false, dev_id);
}
template <typename Device>
inline void DeleteStream(Stream<Device> *stream);

/*! \brief allocate obj->dptr_ for obj->shape_; with pad, rows get an aligned pitch */
template <int dim, typename DType>
inline void AllocSpace(Tensor<cpu, dim, DType> *obj, bool pad = MSHADOW_ALLOC_PAD);
template <int dim, typename DType>
inline void AllocSpace(Tensor<gpu, dim, DType> *obj, bool pad = MSHADOW_ALLOC_PAD);
template <int dim, typename DType>
inline void FreeSpace(Tensor<cpu, dim, DType> *obj);
template <int dim, typename DType>
inline void FreeSpace(Tensor<gpu, dim, DType> *obj);
/*! \brief allocate and fill with initv */
template <typename Device, typename DType, int dim>
inline Tensor<Device, dim, DType> NewTensor(const Shape<dim> &shape, DType initv,
                                            bool pad = MSHADOW_ALLOC_PAD,
                                            Stream<Device> *stream = NULL);

/*! \brief pitch-aware copy between tensors of equal shape, asynchronous on stream for
 *  the GPU forms (synchronous if stream is NULL and MSHADOW_FORCE_STREAM is 0) */
template <int dim, typename DType>
inline void Copy(Tensor<cpu, dim, DType> dst, const Tensor<cpu, dim, DType> &src,
                 Stream<cpu> *stream = NULL);
template <int dim, typename DType>
inline void Copy(Tensor<cpu, dim, DType> dst, const Tensor<gpu, dim, DType> &src,
                 Stream<gpu> *stream = NULL);
template <int dim, typename DType>
inline void Copy(Tensor<gpu, dim, DType> dst, const Tensor<cpu, dim, DType> &src,
                 Stream<gpu> *stream = NULL);
template <int dim, typename DType>
inline void Copy(Tensor<gpu, dim, DType> dst, const Tensor<gpu, dim, DType> &src,
                 Stream<gpu> *stream = NULL);

/*! \brief dst[y] = softmax(energy[y]) for every row */
template <typename DType>
inline void Softmax(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &energy);
template <typename DType>
inline void Softmax(Tensor<gpu, 2, DType> dst, const Tensor<gpu, 2, DType> &energy);
/*! \brief dst = src with 1 subtracted at column label[y] of each row */
template <typename DType>
inline void SoftmaxGrad(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 2, DType> &src,
                        const Tensor<cpu, 1, DType> &label);
template <typename DType>
inline void SoftmaxGrad(const Tensor<gpu, 2, DType> &dst, const Tensor<gpu, 2, DType> &src,
                        const Tensor<gpu, 1, DType> &label);

/*! \brief the rest of the softmax family: label smoothing (alpha), ignore_label, and
 *  3-D tensors (d0, d1, d2) whose softmax runs over the middle dimension */
template <typename DType>
inline void Softmax(Tensor<cpu, 3, DType> dst, const Tensor<cpu, 3, DType> &energy);
template <typename DType>
inline void Softmax(Tensor<gpu, 3, DType> dst, const Tensor<gpu, 3, DType> &energy);
#define MSHADOW_DECLARE_GRAD_FAMILY(Device, DstQual)                                              \
  template <typename DType>                                                                       \
  inline void SmoothSoftmaxGrad(DstQual(Device, 2) dst, const Tensor<Device, 2, DType> &src,      \
                                const Tensor<Device, 1, DType> &label, const float alpha);        \
  template <typename DType>                                                                       \
  inline void SoftmaxGrad(DstQual(Device, 2) dst, const Tensor<Device, 2, DType> &src,            \
                          const Tensor<Device, 1, DType> &label, const DType &ignore_label);      \
  template <typename DType>                                                                       \
  inline void SmoothSoftmaxGrad(DstQual(Device, 2) dst, const Tensor<Device, 2, DType> &src,      \
                                const Tensor<Device, 1, DType> &label, const DType &ignore_label, \
                                const float alpha);                                               \
  template <typename DType>                                                                       \
  inline void SoftmaxGrad(DstQual(Device, 3) dst, const Tensor<Device, 3, DType> &src,            \
                          const Tensor<Device, 2, DType> &label);                                 \
  template <typename DType>                                                                       \
  inline void SmoothSoftmaxGrad(DstQual(Device, 3) dst, const Tensor<Device, 3, DType> &src,      \
                                const Tensor<Device, 2, DType> &label, const float alpha);        \
  template <typename DType>                                                                       \
  inline void SoftmaxGrad(DstQual(Device, 3) dst, const Tensor<Device, 3, DType> &src,            \
                          const Tensor<Device, 2, DType> &label, const DType &ignore_label);      \
  template <typename DType>                                                                       \
  inline void SmoothSoftmaxGrad(DstQual(Device, 3) dst, const Tensor<Device, 3, DType> &src,      \
                                const Tensor<Device, 2, DType> &label, const DType &ignore_label, \
                                const float alpha);
#define MSHADOW_DST_BY_VALUE(Device, dim) Tensor<Device, dim, DType>
#define MSHADOW_DST_BY_CREF(Device, dim) const Tensor<Device, dim, DType> &
MSHADOW_DECLARE_GRAD_FAMILY(cpu, MSHADOW_DST_BY_VALUE)
MSHADOW_DECLARE_GRAD_FAMILY(gpu, MSHADOW_DST_BY_CREF)
#undef MSHADOW_DECLARE_GRAD_FAMILY
#undef MSHADOW_DST_BY_VALUE
#undef MSHADOW_DST_BY_CREF
/*! \brief rows gathered / scattered by an index vector, applied front to back */
template <typename IndexType, typename DType>
inline void AddTakeGrad(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 1, IndexType> &index,
                        const Tensor<cpu, 2, DType> &src);
template <typename IndexType, typename DType>
inline void AddTakeGrad(Tensor<gpu, 2, DType> dst, const Tensor<gpu, 1, IndexType> &index,
                        const Tensor<gpu, 2, DType> &src);
template <typename IndexType, typename DType>
inline void AddTakeGradLargeBatch(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 1, IndexType> &sorted,
                                  const Tensor<cpu, 1, IndexType> &index,
                                  const Tensor<cpu, 2, DType> &src);
template <typename IndexType, typename DType>
inline void AddTakeGradLargeBatch(Tensor<gpu, 2, DType> dst, const Tensor<gpu, 1, IndexType> &sorted,
                                  const Tensor<gpu, 1, IndexType> &index,
                                  const Tensor<gpu, 2, DType> &src);
template <typename IndexType, typename DType>
inline void IndexFill(Tensor<cpu, 2, DType> dst, const Tensor<cpu, 1, IndexType> &index,
                      const Tensor<cpu, 2, DType> &src);
template <typename IndexType, typename DType>
inline void IndexFill(Tensor<gpu, 2, DType> dst, const Tensor<gpu, 1, IndexType> &index,
                      const Tensor<gpu, 2, DType> &src);
/*! \brief stable sort of the (key, value) pairs by key, in place; equivalent keys keep their
 *  order whichever the direction */
template <typename KDType, typename VDType>
inline void SortByKey(Tensor<cpu, 1, KDType> keys, Tensor<cpu, 1, VDType> values,
                      bool is_ascend = true);
template <typename KDType, typename VDType>
inline void SortByKey(Tensor<gpu, 1, KDType> keys, Tensor<gpu, 1, VDType> values,
                      bool is_ascend = true);
/*! \brief ascending sort of the values inside every segment; `segments` is a non-decreasing
 *  vector of segment numbers such as [0, 0, 0, 1, 1, 2, 3, 3] */
template <typename Device, typename VDType, typename SDType>
inline void VectorizedSort(Tensor<Device, 1, VDType> values, Tensor<Device, 1, SDType> segments);

/*! \brief dst[0] = sum_i lhs[i] * rhs[i]; dst is a vector of length one on the same device */
template <typename Device, typename DType>
inline void VectorDot(Tensor<Device, 1, DType> dst, const Tensor<Device, 1, DType> &lhs,
                      const Tensor<Device, 1, DType> &rhs);
/*! \brief dst[b] = alpha * op(lhs[b]) op(rhs[b]) + beta * dst[b] for every matrix b of the batch */
template <bool transpose_left, bool transpose_right, typename Device, typename DType>
inline void BatchGEMM(Tensor<Device, 3, DType> dst, const Tensor<Device, 3, DType> &lhs,
                      const Tensor<Device, 3, DType> &rhs, DType alpha, DType beta,
                      Tensor<Device, 1, DType *> workspace);

/*! \brief Saver::Save(dst(y,x), exp(y,x)) for every element */
template <typename Saver, typename R, int dim, typename DType, typename E, int etype>
inline void MapExp(TRValue<R, cpu, dim, DType> *dst, const expr::Exp<E, DType, etype> &exp);
template <typename Saver, typename R, int dim, typename DType, typename E, int etype>
inline void MapExp(TRValue<R, gpu, dim, DType> *dst, const expr::Exp<E, DType, etype> &exp);
/*! \brief dst[x] <saver>= scale * reduce over rows of exp(y, x) */
template <typename Saver, typename Reducer, typename R, typename DType, typename E, int etype>
inline void MapReduceKeepLowest(TRValue<R, cpu, 1, DType> *dst,
                                const expr::Exp<E, DType, etype> &exp, DType scale = 1);
template <typename Saver, typename Reducer, typename R, typename DType, typename E, int etype>
inline void MapReduceKeepLowest(TRValue<R, gpu, 1, DType> *dst,
                                const expr::Exp<E, DType, etype> &exp, DType scale = 1);
/*! \brief dst[c] <saver>= scale * reduce over every dimension but dimkeep */
template <typename Saver, typename Reducer, int dimkeep, typename R, typename DType, typename E,
          int etype>
inline void MapReduceKeepHighDim(TRValue<R, cpu, 1, DType> *dst,
                                 const expr::Exp<E, DType, etype> &exp, DType scale = 1);
template <typename Saver, typename Reducer, int dimkeep, typename R, typename DType, typename E,
          int etype>
inline void MapReduceKeepHighDim(TRValue<R, gpu, 1, DType> *dst,
                                 const expr::Exp<E, DType, etype> &exp, DType scale = 1);

}  // namespace mshadow

#include "./expr/engine.h"
#include "./extension.h"
#include "./expr/scalar_ops.h"
#include "./cpu/tensor_cpu.h"
#include "./hip/tensor_gpu.h"
#include "./dot_engine.h"
#include "./io.h"
#include "./tensor_container.h"
#include "./random.h"

#endif  // MSHADOW_TENSOR_H_
