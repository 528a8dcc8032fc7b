/*
 * Tensor<gpu>: the gfx950 device of the API.
 *
 * Host-side definitions that replace mshadow/tensor_gpu-inl.h:14-214 of the reference.
 * Memory, copies, streams and the fixed-function operations go through the C ABI of
 * libmshadow_hip (include/mshadow_hip.h) and are available to any translation unit.
 * Evaluating an arbitrary expression into a Tensor<gpu> instantiates a kernel template
 * from mshadow/hip/kernels/ for the caller's expression type and starts it through
 * mshadow_hip_launch; that part needs hipcc, exactly as the reference needs nvcc for
 * it (tensor_gpu-inl.h:96-98). Expressions whose shape the library knows - pool /
 * unpool of float tensors, unpack_patch2col(pad(tensor)), crop(pack_col2patch(tensor)),
 * reductions of plain float tensors - are routed to the tuned fixed-function kernels
 * first (FastPath below).
 */
#ifndef MSHADOW_HIP_TENSOR_GPU_H_
#define MSHADOW_HIP_TENSOR_GPU_H_

#include <mshadow_hip.h>

#include <cstring>

#include "../tensor.h"
#include "./stream.h"

#if defined(__HIPCC__)
#include "./kernels/map.h"
#include "./kernels/reduce.h"
#include "./kernels/reduce_dma.h"
#include "./kernels/rows_by_index.h"
#include "./kernels/softmax_any.h"
#include "./kernels/sort_any.h"
#endif

namespace mshadow {

template <>
inline void InitTensorEngine<gpu>(int dev_id) {
  int device_count = 0;
  MSHADOW_HIP_CALL(mshadow_hip_device_count(&device_count));
  CHECK_GT(device_count, 0) << "Cannot find a HIP device. Please check the ROCm installation";
  const int device_id = dev_id < 0 ? 0 : dev_id;
  CHECK_LT(device_id, device_count) << "Incorrect Device ID";
  MSHADOW_HIP_CALL(mshadow_hip_set_device(device_id));
  mshadow_hip_props prop;
  MSHADOW_HIP_CALL(mshadow_hip_get_props(device_id, &prop));
}
template <>
inline void ShutdownTensorEngine<gpu>(void) {}
template <>
inline void SetDevice<gpu>(int devid) {
  MSHADOW_HIP_CALL(mshadow_hip_set_device(devid));
}

/*! \brief pinned host memory for transfers */
template <>
inline void *AllocHost_<gpu>(size_t size) {
  void *dptr;
  MSHADOW_HIP_CALL(mshadow_hip_malloc_host(&dptr, size));
  return dptr;
}
template <>
inline void FreeHost_<gpu>(void *dptr) {
  MSHADOW_HIP_CALL(mshadow_hip_free_host(dptr));
}

/*! \brief rows get a 256-byte-aligned pitch when padding is on and the last dimension
 *  is at least MSHADOW_MIN_PAD_RATIO * 32 elements (rule of tensor_gpu-inl.h:37-51) */
template <int dim, typename DType>
inline void AllocSpace(Tensor<gpu, dim, DType> *obj, bool pad) {
  size_t pitch;
  void *p = NULL;
  if (pad && obj->size(dim - 1) >= MSHADOW_MIN_PAD_RATIO * 32) {
    MSHADOW_HIP_CALL(mshadow_hip_malloc_pitch(&p, &pitch, obj->size(dim - 1) * sizeof(DType),
                                              obj->shape_.FlatTo2D()[0]));
    obj->stride_ = static_cast<index_t>(pitch / sizeof(DType));
  } else {
    obj->stride_ = obj->size(dim - 1);
    MSHADOW_HIP_CALL(mshadow_hip_malloc_pitch(&p, &pitch, obj->shape_.Size() * sizeof(DType), 1));
  }
  obj->dptr_ = reinterpret_cast<DType *>(p);
}
template <int dim, typename DType>
inline void FreeSpace(Tensor<gpu, dim, DType> *obj) {
  MSHADOW_HIP_CALL(mshadow_hip_free(obj->dptr_));
  obj->dptr_ = NULL;
}

namespace gpu_detail {
template <typename A, typename B, int dim, typename DType>
inline void Copy2D(Tensor<A, dim, DType> _dst, Tensor<B, dim, DType> _src, int kind,
                   Stream<gpu> *stream) {
  CHECK_EQ(_dst.shape_, _src.shape_) << "Copy:shape mismatch";
  Tensor<A, 2, DType> dst = _dst.FlatTo2D();
  Tensor<B, 2, DType> src = _src.FlatTo2D();
  MSHADOW_HIP_CALL(mshadow_hip_memcpy2d_async(
      dst.dptr_, dst.stride_ * sizeof(DType), src.dptr_, src.stride_ * sizeof(DType),
      dst.size(1) * sizeof(DType), dst.size(0), kind, Stream<gpu>::GetStream(stream)));
  if (stream == NULL) {  // only reachable with MSHADOW_FORCE_STREAM off
    MSHADOW_HIP_CALL(mshadow_hip_stream_sync(NULL));
  }
}
}  // namespace gpu_detail

template <int dim, typename DType>
inline void Copy(Tensor<cpu, dim, DType> dst, const Tensor<gpu, dim, DType> &src,
                 Stream<gpu> *stream) {
  gpu_detail::Copy2D(dst, src, MSHADOW_HIP_D2H, stream);
}
template <int dim, typename DType>
inline void Copy(Tensor<gpu, dim, DType> dst, const Tensor<gpu, dim, DType> &src,
                 Stream<gpu> *stream) {
  gpu_detail::Copy2D(dst, src, MSHADOW_HIP_D2D, stream);
}
template <int dim, typename DType>
inline void Copy(Tensor<gpu, dim, DType> dst, const Tensor<cpu, dim, DType> &src,
                 Stream<gpu> *stream) {
  gpu_detail::Copy2D(dst, src, MSHADOW_HIP_H2D, stream);
}

/* ------------------------------------------------------------------ fixed-function ops */
namespace gpu_detail {
template <typename Saver>
struct SaverCode {
  static const int value = -1;
};
template <>
struct SaverCode<sv::saveto> { static const int value = MSHADOW_HIP_SAVETO; };
template <>
struct SaverCode<sv::plusto> { static const int value = MSHADOW_HIP_PLUSTO; };
template <>
struct SaverCode<sv::minusto> { static const int value = MSHADOW_HIP_MINUSTO; };
template <>
struct SaverCode<sv::multo> { static const int value = MSHADOW_HIP_MULTO; };
template <>
struct SaverCode<sv::divto> { static const int value = MSHADOW_HIP_DIVTO; };
template <typename Reducer>
struct ReducerCode {
  static const int value = -1;
};
template <>
struct ReducerCode<red::sum> { static const int value = MSHADOW_HIP_SUM; };
template <>
struct ReducerCode<red::maximum> { static const int value = MSHADOW_HIP_MAX; };
template <>
struct ReducerCode<red::minimum> { static const int value = MSHADOW_HIP_MIN; };

inline const uint16_t *Bits(const half::half_t *p) { return reinterpret_cast<const uint16_t *>(p); }
inline uint16_t *Bits(half::half_t *p) { return reinterpret_cast<uint16_t *>(p); }
}  // namespace gpu_detail

inline void Softmax(Tensor<gpu, 2, float> dst, const Tensor<gpu, 2, float> &src) {
  CHECK_EQ(dst.shape_, src.shape_) << "Softmax: shape mismatch";
  MSHADOW_HIP_CALL(mshadow_hip_softmax_f32(dst.dptr_, dst.stride_, src.dptr_, src.stride_,
                                           dst.size(0), dst.size(1),
                                           Stream<gpu>::GetStream(dst.stream_)));
}
inline void SoftmaxGrad(const Tensor<gpu, 2, float> &dst, const Tensor<gpu, 2, float> &src,
                        const Tensor<gpu, 1, float> &label) {
  CHECK_EQ(dst.shape_, src.shape_) << "SoftmaxGrad: shape mismatch";
  CHECK_EQ(dst.size(0), label.size(0)) << "SoftmaxGrad: label shape mismatch";
  MSHADOW_HIP_CALL(mshadow_hip_softmax_grad_f32(dst.dptr_, dst.stride_, src.dptr_, src.stride_,
                                                label.dptr_, dst.size(0), dst.size(1),
                                                Stream<gpu>::GetStream(dst.stream_)));
}
/* other element types (half_t, double): kernel templates in the element type's own
   arithmetic, instantiated in the calling translation unit (kernels/softmax_any.h) */
namespace gpu_detail {
/*! \brief rows of whole packs that all start 16-byte aligned: 128-bit accesses */
template <typename DType>
inline bool AnyPackable(const DType *a, uint32_t astride, const DType *b, uint32_t bstride,
                        uint32_t cols, int pack) {
  const size_t addr = reinterpret_cast<size_t>(a) | reinterpret_cast<size_t>(b) |
                      (static_cast<size_t>(astride) * sizeof(DType)) |
                      (static_cast<size_t>(bstride) * sizeof(DType));
  return addr % 16 == 0 && cols % pack == 0;
}
}  // namespace gpu_detail
namespace gpu_detail {
#if defined(__HIPCC__)
/*! \brief long half_t rows: one workgroup per row, the row kept in registers; false = not
 *  this shape or element type */
template <typename DType>
inline bool SoftmaxLongRows(DType *, uint32_t, const DType *, uint32_t, uint32_t, uint32_t, bool, void *) {
  return false;
}
inline bool SoftmaxLongRows(half::half_t *d, uint32_t dstride, const half::half_t *s, uint32_t sstride,
                            uint32_t rows, uint32_t cols, bool vec, void *stream) {
  if (cols < static_cast<uint32_t>(hip::kHalfRowMinCols) ||
      cols > static_cast<uint32_t>(hip::kHalfRowMaxCols)) {
    return false;
  }
  void *args[] = {&d, &dstride, &s, &sstride, &cols};
  const uint32_t grid[3] = {rows, 1, 1};
  const uint32_t block[3] = {static_cast<uint32_t>(hip::kHalfRowBlock), 1, 1};
  const void *kernel = vec ? reinterpret_cast<const void *>(hip::SoftmaxHalfRowKernel<true>)
                           : reinterpret_cast<const void *>(hip::SoftmaxHalfRowKernel<false>);
  MSHADOW_HIP_CALL(mshadow_hip_launch(kernel, grid, block, args, 0, stream));
  return true;
}
#endif
}  // namespace gpu_detail
template <typename DType>
inline void Softmax(Tensor<gpu, 2, DType> dst, const Tensor<gpu, 2, DType> &src) {
  CHECK_EQ(dst.shape_, src.shape_) << "Softmax: shape mismatch";
#if defined(__HIPCC__)
  uint32_t rows = dst.size(0), cols = dst.size(1);
  if (rows == 0 || cols == 0) return;
  DType *d = dst.dptr_;
  const DType *s = src.dptr_;
  uint32_t dstride = dst.stride_, sstride = src.stride_;
  if (gpu_detail::SoftmaxLongRows(d, dstride, s, sstride, rows, cols,
                                  gpu_detail::AnyPackable(s, sstride, const_cast<const DType *>(d),
                                                          dstride, cols, hip::kAnyTile),
                                  Stream<gpu>::GetStream(dst.stream_))) {
    return;
  }
  void *args[] = {&d, &dstride, &s, &sstride, &rows, &cols};
  const uint32_t grid[3] = {(rows + hip::kAnyRows - 1) / hip::kAnyRows, 1, 1};
  const uint32_t block[3] = {static_cast<uint32_t>(hip::kAnyBlock), 1, 1};
  const bool vec = gpu_detail::AnyPackable(s, sstride, const_cast<const DType *>(d), dstride, cols,
                                           hip::kAnyTile);
  const void *kernel = vec ? reinterpret_cast<const void *>(hip::SoftmaxAnyKernel<DType, true>)
                           : reinterpret_cast<const void *>(hip::SoftmaxAnyKernel<DType, false>);
  MSHADOW_HIP_CALL(mshadow_hip_launch(kernel, grid, block, args, 0,
                                      Stream<gpu>::GetStream(dst.stream_)));
#else
  LOG(FATAL) << "Softmax<gpu> of this element type: compile the calling translation unit with hipcc";
#endif
}
namespace gpu_detail {
/*! \brief static_cast<int>(label) as the host makes it (half_t goes through float) */
inline int LabelAsInt(half::half_t v) { return static_cast<int>(static_cast<float>(v)); }
template <typename DType>
inline int LabelAsInt(DType v) { return static_cast<int>(v); }
/*! \brief alpha / (classes - 1), the count converted from unsigned as the host writes it
 *  (mshadow/tensor_cpu-inl.h:308) - a float whatever the element type */
inline float SmoothShare(float alpha, index_t classes) {
  return alpha / static_cast<float>(classes - 1);
}

/*! \brief the 2-D gradients of any element type: flags as MSHADOW_HIP_GRAD_* */
template <typename DType>
inline void AnyGrad2D(const Tensor<gpu, 2, DType> &dst, const Tensor<gpu, 2, DType> &src,
                      const Tensor<gpu, 1, DType> &label, int flags, int ignore_k, float alpha) {
  CHECK_EQ(dst.shape_, src.shape_) << "SoftmaxGrad: shape mismatch";
  CHECK_EQ(dst.size(0), label.size(0)) << "SoftmaxGrad: label shape mismatch";
#if defined(__HIPCC__)
  uint32_t rows = dst.size(0), cols = dst.size(1);
  if (rows == 0 || cols == 0) return;
  DType *d = dst.dptr_;
  const DType *s = src.dptr_;
  const DType *l = label.dptr_;
  uint32_t dstride = dst.stride_, sstride = src.stride_;
  float smooth = SmoothShare(alpha, dst.size(1));
  void *args[] = {&d, &dstride, &s, &sstride, &l, &cols, &ignore_k, &alpha, &smooth};
  /* rows on the grid's x axis (up to 2^31 - 1), a row's packs over a few workgroups */
  const uint32_t per_block = hip::kAnyBlock * hip::kAnyTile;
  uint32_t per_row = (cols + per_block - 1) / per_block;
  if (per_row > 64) per_row = 64;
  const uint32_t grid[3] = {rows, per_row, 1};
  const uint32_t block[3] = {static_cast<uint32_t>(hip::kAnyBlock), 1, 1};
  const bool vec = AnyPackable(s, sstride, const_cast<const DType *>(d), dstride, cols,
                               hip::kAnyTile);
  const void *kernel = NULL;
#define MSHADOW_ANY_GRAD(FLAGS)                                                              \
  kernel = vec ? reinterpret_cast<const void *>(hip::SoftmaxGradAnyKernel<DType, true, FLAGS>) \
               : reinterpret_cast<const void *>(hip::SoftmaxGradAnyKernel<DType, false, FLAGS>)
  switch (flags) {
    case 0: MSHADOW_ANY_GRAD(0); break;
    case 1: MSHADOW_ANY_GRAD(1); break;
    case 2: MSHADOW_ANY_GRAD(2); break;
    default: MSHADOW_ANY_GRAD(3); break;
  }
#undef MSHADOW_ANY_GRAD
  MSHADOW_HIP_CALL(mshadow_hip_launch(kernel, grid, block, args, 0,
                                      Stream<gpu>::GetStream(dst.stream_)));
#else
  LOG(FATAL) << "SoftmaxGrad<gpu> of this element type: compile the calling translation unit with hipcc";
#endif
}

/*! \brief the 3-D gradients of any element type */
template <typename DType>
inline void AnyGrad3D(const Tensor<gpu, 3, DType> &dst, const Tensor<gpu, 3, DType> &src,
                      const Tensor<gpu, 2, DType> &label, int flags, int ignore_k, float alpha) {
  CHECK_EQ(dst.shape_, src.shape_) << "SoftmaxGrad: shape mismatch";
  CHECK(dst.size(0) == label.size(0) && dst.size(2) == label.size(1))
      << "SoftmaxGrad: label shape mismatch";
#if defined(__HIPCC__)
  uint32_t d0 = dst.size(0), d1 = dst.size(1), d2 = dst.size(2);
  if (d0 == 0 || d1 == 0 || d2 == 0) return;
  DType *d = dst.dptr_;
  const DType *s = src.dptr_;
  const DType *l = label.dptr_;
  uint32_t dstride = dst.stride_, sstride = src.stride_, lstride = label.stride_;
  float smooth = SmoothShare(alpha, dst.size(1));
  void *args[] = {&d, &dstride, &s, &sstride, &l, &lstride, &d0, &d1, &d2, &ignore_k, &alpha, &smooth};
  const size_t total = static_cast<size_t>(d0) * d1 * d2;
  size_t blocks = (total + hip::kAny3dBlock - 1) / hip::kAny3dBlock;
  if (blocks > (1u << 20)) blocks = 1u << 20;  // the kernel strides over what is left
  const uint32_t grid[3] = {static_cast<uint32_t>(blocks), 1, 1};
  const uint32_t block[3] = {static_cast<uint32_t>(hip::kAny3dBlock), 1, 1};
  const void *kernel = NULL;
  switch (flags) {
    case 0: kernel = reinterpret_cast<const void *>(hip::SoftmaxGrad3dAnyKernel<DType, 0>); break;
    case 1: kernel = reinterpret_cast<const void *>(hip::SoftmaxGrad3dAnyKernel<DType, 1>); break;
    case 2: kernel = reinterpret_cast<const void *>(hip::SoftmaxGrad3dAnyKernel<DType, 2>); break;
    default: kernel = reinterpret_cast<const void *>(hip::SoftmaxGrad3dAnyKernel<DType, 3>); break;
  }
  MSHADOW_HIP_CALL(mshadow_hip_launch(kernel, grid, block, args, 0,
                                      Stream<gpu>::GetStream(dst.stream_)));
#else
  LOG(FATAL) << "SoftmaxGrad<gpu> of this element type: compile the calling translation unit with hipcc";
#endif
}

/*! \brief AddTakeGrad (OP 0) / AddTakeGradLargeBatch (1) / IndexFill (2) of any element and
 *  index type: the kernel of mshadow/hip/kernels/rows_by_index.h compiled with the caller */
template <int OP, typename IndexType, typename DType>
inline void AnyRowsByIndex(Tensor<gpu, 2, DType> dst, const Tensor<gpu, 1, IndexType> &rows_of,
                           const Tensor<gpu, 1, IndexType> &from_of,
                           const Tensor<gpu, 2, DType> &src) {
#if defined(__HIPCC__)
  int k_rows = dst.size(0), n_index = from_of.size(0), cols = dst.size(1);
  if (k_rows == 0 || n_index == 0 || cols == 0) return;
  CHECK_LT(static_cast<uint64_t>(k_rows) + 1024u * 16u, 1ull << 31) << "table too tall";
  DType *d = dst.dptr_;
  const DType *s = src.dptr_;
  const IndexType *r = rows_of.dptr_;
  const IndexType *f = from_of.dptr_;
  int dstride = dst.stride_, sstride = src.stride_, rows_per_wave = 0;
  unsigned blocks = 0;
  hip::RowsByIndexGrid(k_rows, &blocks, &rows_per_wave);
  void *args[] = {&d, &dstride, &k_rows, &rows_per_wave, &r, &f, &n_index, &s, &sstride, &cols};
  const uint32_t grid[3] = {blocks, 1, 1};
  const uint32_t block[3] = {static_cast<uint32_t>(hip::kTakeBlock), 1, 1};
  MSHADOW_HIP_CALL(mshadow_hip_launch(
      reinterpret_cast<const void *>(hip::RowsByIndexKernel<IndexType, DType, OP, false>), grid,
      block, args, 0, Stream<gpu>::GetStream(dst.stream_)));
#else
  LOG(FATAL) << "row scatter of this element type: compile the calling translation unit with hipcc";
#endif
}
/*! \brief which implementation a row scatter takes: float tables with int32 or float index
 *  vectors call the library's fixed-function kernels, everything else the template above */
template <typename IndexType, typename DType>
struct RowsByIndexRoute {
  inline static void Run(int op, Tensor<gpu, 2, DType> dst, const Tensor<gpu, 1, IndexType> &rows_of,
                         const Tensor<gpu, 1, IndexType> &from_of, const Tensor<gpu, 2, DType> &src) {
    if (op == 0) AnyRowsByIndex<0>(dst, rows_of, from_of, src);
    else if (op == 1) AnyRowsByIndex<1>(dst, rows_of, from_of, src);
    else AnyRowsByIndex<2>(dst, rows_of, from_of, src);
  }
};
template <typename IndexType, int IS_INT>
struct RowsByIndexLibrary {
  inline static void Run(int op, Tensor<gpu, 2, float> dst, const Tensor<gpu, 1, IndexType> &rows_of,
                         const Tensor<gpu, 1, IndexType> &from_of, const Tensor<gpu, 2, float> &src) {
    void *stream = Stream<gpu>::GetStream(dst.stream_);
    if (op == 0) {
      MSHADOW_HIP_CALL(mshadow_hip_add_take_grad_f32(dst.dptr_, dst.stride_, dst.size(0), from_of.dptr_,
                                                     IS_INT, from_of.size(0), src.dptr_, src.stride_,
                                                     src.size(1), stream));
    } else if (op == 1) {
      MSHADOW_HIP_CALL(mshadow_hip_add_take_grad_large_batch_f32(
          dst.dptr_, dst.stride_, dst.size(0), rows_of.dptr_, from_of.dptr_, IS_INT, from_of.size(0),
          src.dptr_, src.stride_, src.size(1), stream));
    } else {
      MSHADOW_HIP_CALL(mshadow_hip_index_fill_f32(dst.dptr_, dst.stride_, dst.size(0), from_of.dptr_,
                                                  IS_INT, from_of.size(0), src.dptr_, src.stride_,
                                                  src.size(1), stream));
    }
  }
};
template <>
struct RowsByIndexRoute<int, float> : public RowsByIndexLibrary<int, 1> {};
template <>
struct RowsByIndexRoute<float, float> : public RowsByIndexLibrary<float, 0> {};
}  // namespace gpu_detail

/* ---- the softmax family for any element type (mshadow/tensor_gpu-inl.h:157-215): kernels in
 * the element type's own arithmetic, compiled with the caller. Float tensors take the
 * non-template overloads further down, which call the library. */
template <typename DType>
inline void SoftmaxGrad(const Tensor<gpu, 2, DType> &dst, const Tensor<gpu, 2, DType> &src,
                        const Tensor<gpu, 1, DType> &label) {
  gpu_detail::AnyGrad2D(dst, src, label, 0, 0, 0.0f);
}
template <typename DType>
inline void SmoothSoftmaxGrad(const Tensor<gpu, 2, DType> &dst, const Tensor<gpu, 2, DType> &src,
                              const Tensor<gpu, 1, DType> &label, const float alpha) {
  gpu_detail::AnyGrad2D(dst, src, label, MSHADOW_HIP_GRAD_SMOOTH, 0, alpha);
}
template <typename DType>
inline void SoftmaxGrad(const Tensor<gpu, 2, DType> &dst, const Tensor<gpu, 2, DType> &src,
                        const Tensor<gpu, 1, DType> &label, const DType &ignore_label) {
  gpu_detail::AnyGrad2D(dst, src, label, MSHADOW_HIP_GRAD_IGNORE,
                        gpu_detail::LabelAsInt(ignore_label), 0.0f);
}
template <typename DType>
inline void SmoothSoftmaxGrad(const Tensor<gpu, 2, DType> &dst, const Tensor<gpu, 2, DType> &src,
                              const Tensor<gpu, 1, DType> &label, const DType &ignore_label,
                              const float alpha) {
  gpu_detail::AnyGrad2D(dst, src, label, MSHADOW_HIP_GRAD_SMOOTH | MSHADOW_HIP_GRAD_IGNORE,
                        gpu_detail::LabelAsInt(ignore_label), alpha);
}
template <typename DType>
inline void Softmax(Tensor<gpu, 3, DType> dst, const Tensor<gpu, 3, DType> &src) {
  CHECK_EQ(dst.shape_, src.shape_) << "Softmax: shape mismatch";
#if defined(__HIPCC__)
  uint32_t d0 = dst.size(0), d1 = dst.size(1), d2 = dst.size(2);
  if (d0 == 0 || d1 == 0 || d2 == 0) return;
  DType *d = dst.dptr_;
  const DType *s = src.dptr_;
  uint32_t dstride = dst.stride_, sstride = src.stride_;
  void *args[] = {&d, &dstride, &s, &sstride, &d0, &d1, &d2};
  const size_t columns = static_cast<size_t>(d0) * d2;
  CHECK_LT(columns, (1ull << 31) * hip::kAny3dBlock) << "Softmax: too many columns";
  const uint32_t grid[3] = {static_cast<uint32_t>((columns + hip::kAny3dBlock - 1) / hip::kAny3dBlock), 1, 1};
  const uint32_t block[3] = {static_cast<uint32_t>(hip::kAny3dBlock), 1, 1};
  MSHADOW_HIP_CALL(mshadow_hip_launch(reinterpret_cast<const void *>(hip::Softmax3dAnyKernel<DType>),
                                      grid, block, args, 0, Stream<gpu>::GetStream(dst.stream_)));
#else
  LOG(FATAL) << "Softmax<gpu> of this element type: compile the calling translation unit with hipcc";
#endif
}
template <typename DType>
inline void SoftmaxGrad(const Tensor<gpu, 3, DType> &dst, const Tensor<gpu, 3, DType> &src,
                        const Tensor<gpu, 2, DType> &label) {
  gpu_detail::AnyGrad3D(dst, src, label, 0, 0, 0.0f);
}
template <typename DType>
inline void SmoothSoftmaxGrad(const Tensor<gpu, 3, DType> &dst, const Tensor<gpu, 3, DType> &src,
                              const Tensor<gpu, 2, DType> &label, const float alpha) {
  gpu_detail::AnyGrad3D(dst, src, label, MSHADOW_HIP_GRAD_SMOOTH, 0, alpha);
}
template <typename DType>
inline void SoftmaxGrad(const Tensor<gpu, 3, DType> &dst, const Tensor<gpu, 3, DType> &src,
                        const Tensor<gpu, 2, DType> &label, const DType &ignore_label) {
  gpu_detail::AnyGrad3D(dst, src, label, MSHADOW_HIP_GRAD_IGNORE,
                        gpu_detail::LabelAsInt(ignore_label), 0.0f);
}
template <typename DType>
inline void SmoothSoftmaxGrad(const Tensor<gpu, 3, DType> &dst, const Tensor<gpu, 3, DType> &src,
                              const Tensor<gpu, 2, DType> &label, const DType &ignore_label,
                              const float alpha) {
  gpu_detail::AnyGrad3D(dst, src, label, MSHADOW_HIP_GRAD_SMOOTH | MSHADOW_HIP_GRAD_IGNORE,
                        gpu_detail::LabelAsInt(ignore_label), alpha);
}
/* ---- the row scatter / gather functions for any element and index type
 * (mshadow/tensor_gpu-inl.h:217-240); float tensors with int32 or float indices take the
 * overloads further down */
template <typename IndexType, typename DType>
inline void AddTakeGrad(Tensor<gpu, 2, DType> dst, const Tensor<gpu, 1, IndexType> &index,
                        const Tensor<gpu, 2, DType> &src) {
  CHECK_EQ(dst.size(1), src.size(1)) << "AddTakeGrad: shape mismatch";
  CHECK_EQ(index.size(0), src.size(0)) << "AddTakeGrad: shape mismatch";
  gpu_detail::RowsByIndexRoute<IndexType, DType>::Run(0, dst, index, index, src);
}
template <typename IndexType, typename DType>
inline void AddTakeGradLargeBatch(Tensor<gpu, 2, DType> dst, const Tensor<gpu, 1, IndexType> &sorted,
                                  const Tensor<gpu, 1, IndexType> &index,
                                  const Tensor<gpu, 2, DType> &src) {
  CHECK_EQ(dst.size(1), src.size(1)) << "AddTakeGradLargeBatch: shape mismatch";
  CHECK_EQ(sorted.size(0), index.size(0)) << "AddTakeGradLargeBatch: shape mismatch";
  gpu_detail::RowsByIndexRoute<IndexType, DType>::Run(1, dst, sorted, index, src);
}
template <typename IndexType, typename DType>
inline void IndexFill(Tensor<gpu, 2, DType> dst, const Tensor<gpu, 1, IndexType> &index,
                      const Tensor<gpu, 2, DType> &src) {
  CHECK_EQ(dst.size(1), src.size(1)) << "IndexFill: shape mismatch";
  CHECK_EQ(index.size(0), src.size(0)) << "IndexFill: shape mismatch";
  gpu_detail::RowsByIndexRoute<IndexType, DType>::Run(2, dst, index, index, src);
}

/* ---- the softmax family for float tensors: non-template overloads, each one call into the
 * library's fixed-function kernels */
namespace gpu_detail {
inline void Grad2D(const Tensor<gpu, 2, float> &dst, const Tensor<gpu, 2, float> &src,
                   const Tensor<gpu, 1, float> &label, int flags, float ignore_label, float alpha) {
  CHECK_EQ(dst.shape_, src.shape_) << "SoftmaxGrad: shape mismatch";
  CHECK_EQ(dst.size(0), label.size(0)) << "SoftmaxGrad: label shape mismatch";
  MSHADOW_HIP_CALL(mshadow_hip_softmax_grad_ex_f32(
      dst.dptr_, dst.stride_, src.dptr_, src.stride_, label.dptr_, dst.size(0), dst.size(1), flags,
      ignore_label, alpha, Stream<gpu>::GetStream(dst.stream_)));
}
inline void Grad3D(const Tensor<gpu, 3, float> &dst, const Tensor<gpu, 3, float> &src,
                   const Tensor<gpu, 2, float> &label, int flags, float ignore_label, float alpha) {
  CHECK_EQ(dst.shape_, src.shape_) << "SoftmaxGrad: shape mismatch";
  CHECK(dst.size(0) == label.size(0) && dst.size(2) == label.size(1))
      << "SoftmaxGrad: label shape mismatch";
  MSHADOW_HIP_CALL(mshadow_hip_softmax3d_grad_f32(
      dst.dptr_, dst.stride_, src.dptr_, src.stride_, label.dptr_, label.stride_, dst.size(0),
      dst.size(1), dst.size(2), flags, ignore_label, alpha, Stream<gpu>::GetStream(dst.stream_)));
}
}  // namespace gpu_detail

inline void Softmax(Tensor<gpu, 3, float> dst, const Tensor<gpu, 3, float> &src) {
  CHECK_EQ(dst.shape_, src.shape_) << "Softmax: shape mismatch";
  MSHADOW_HIP_CALL(mshadow_hip_softmax3d_f32(dst.dptr_, dst.stride_, src.dptr_, src.stride_,
                                             dst.size(0), dst.size(1), dst.size(2),
                                             Stream<gpu>::GetStream(dst.stream_)));
}
inline void SmoothSoftmaxGrad(const Tensor<gpu, 2, float> &dst, const Tensor<gpu, 2, float> &src,
                              const Tensor<gpu, 1, float> &label, const float alpha) {
  gpu_detail::Grad2D(dst, src, label, MSHADOW_HIP_GRAD_SMOOTH, 0.0f, alpha);
}
inline void SoftmaxGrad(const Tensor<gpu, 2, float> &dst, const Tensor<gpu, 2, float> &src,
                        const Tensor<gpu, 1, float> &label, const float &ignore_label) {
  gpu_detail::Grad2D(dst, src, label, MSHADOW_HIP_GRAD_IGNORE, ignore_label, 0.0f);
}
inline void SmoothSoftmaxGrad(const Tensor<gpu, 2, float> &dst, const Tensor<gpu, 2, float> &src,
                              const Tensor<gpu, 1, float> &label, const float &ignore_label,
                              const float alpha) {
  gpu_detail::Grad2D(dst, src, label, MSHADOW_HIP_GRAD_SMOOTH | MSHADOW_HIP_GRAD_IGNORE,
                     ignore_label, alpha);
}
inline void SoftmaxGrad(const Tensor<gpu, 3, float> &dst, const Tensor<gpu, 3, float> &src,
                        const Tensor<gpu, 2, float> &label) {
  gpu_detail::Grad3D(dst, src, label, 0, 0.0f, 0.0f);
}
inline void SmoothSoftmaxGrad(const Tensor<gpu, 3, float> &dst, const Tensor<gpu, 3, float> &src,
                              const Tensor<gpu, 2, float> &label, const float alpha) {
  gpu_detail::Grad3D(dst, src, label, MSHADOW_HIP_GRAD_SMOOTH, 0.0f, alpha);
}
inline void SoftmaxGrad(const Tensor<gpu, 3, float> &dst, const Tensor<gpu, 3, float> &src,
                        const Tensor<gpu, 2, float> &label, const float &ignore_label) {
  gpu_detail::Grad3D(dst, src, label, MSHADOW_HIP_GRAD_IGNORE, ignore_label, 0.0f);
}
inline void SmoothSoftmaxGrad(const Tensor<gpu, 3, float> &dst, const Tensor<gpu, 3, float> &src,
                              const Tensor<gpu, 2, float> &label, const float &ignore_label,
                              const float alpha) {
  gpu_detail::Grad3D(dst, src, label, MSHADOW_HIP_GRAD_SMOOTH | MSHADOW_HIP_GRAD_IGNORE,
                     ignore_label, alpha);
}
namespace gpu_detail {
/*! \brief how the bits of a 32-bit key type are ordered (-1: no device sort for this type) */
template <typename KDType>
struct SortKeyKind { static const int value = -1; };
template <>
struct SortKeyKind<float> { static const int value = MSHADOW_HIP_KEY_F32; };
template <>
struct SortKeyKind<int32_t> { static const int value = MSHADOW_HIP_KEY_I32; };
template <>
struct SortKeyKind<uint32_t> { static const int value = MSHADOW_HIP_KEY_U32; };
/*! \brief device memory that is given back when its owner goes out of scope - also when a
 *  failed call between allocation and release throws (DMLC_LOG_FATAL_THROW builds) */
struct ScopedDeviceBlock {
  void *ptr;
  ScopedDeviceBlock() : ptr(NULL) {}
  ~ScopedDeviceBlock() {
    if (ptr != NULL) (void)mshadow_hip_free(ptr);
  }
  inline void Allocate(size_t bytes) {
    size_t pitch = 0;
    MSHADOW_HIP_CALL(mshadow_hip_malloc_pitch(&ptr, &pitch, bytes, 1));
  }
  inline void Release() {
    void *p = ptr;
    ptr = NULL;
    MSHADOW_HIP_CALL(mshadow_hip_free(p));
  }

 private:
  ScopedDeviceBlock(const ScopedDeviceBlock &);
  ScopedDeviceBlock &operator=(const ScopedDeviceBlock &);
};
/*! \brief the device sort for key / value types the library's 32-bit entry point does not
 *  take: through a permutation, one stable 32-bit pass per key word (kernels/sort_any.h) */
template <typename KDType, typename VDType>
inline void SortByKeyThroughPermutation(Tensor<gpu, 1, KDType> keys, Tensor<gpu, 1, VDType> values,
                                        bool is_ascend) {
#if defined(__HIPCC__)
  const size_t n = keys.size(0);
  CHECK_LT(n, 1ull << 31) << "SortByKey: too many elements";
  void *stream = Stream<gpu>::GetStream(keys.stream_);
  size_t sort_bytes = 0;
  MSHADOW_HIP_CALL(mshadow_hip_sort_by_key_workspace(n, &sort_bytes));
  /* words | permutation | copy of the keys | copy of the values | the sort's scratch, each
     part starting on a multiple of 256 bytes */
  const size_t part = 256;
  const size_t words_at = 0;
  const size_t perm_at = words_at + (n * 4 + part - 1) / part * part;
  const size_t keys_at = perm_at + (n * 4 + part - 1) / part * part;
  const size_t vals_at = keys_at + (n * sizeof(KDType) + part - 1) / part * part;
  const size_t sort_at = vals_at + (n * sizeof(VDType) + part - 1) / part * part;
  ScopedDeviceBlock block;
  block.Allocate(sort_at + sort_bytes);
  char *base = static_cast<char *>(block.ptr);
  uint32_t *words = reinterpret_cast<uint32_t *>(base + words_at);
  uint32_t *perm = reinterpret_cast<uint32_t *>(base + perm_at);
  KDType *keys_copy = reinterpret_cast<KDType *>(base + keys_at);
  VDType *vals_copy = reinterpret_cast<VDType *>(base + vals_at);
  uint32_t count = static_cast<uint32_t>(n);
  uint32_t blocks = (count + hip::kSortAnyBlock - 1) / hip::kSortAnyBlock;
  if (blocks > 65536u) blocks = 65536u;
  const uint32_t grid[3] = {blocks, 1, 1};
  const uint32_t block_dim[3] = {static_cast<uint32_t>(hip::kSortAnyBlock), 1, 1};
  const KDType *key_src = keys.dptr_;
  const uint32_t *no_perm = NULL;
  const uint32_t *cur_perm = perm;
  {  // low word of every key, and the identity permutation
    void *args[] = {&words, &perm, &key_src, &no_perm, &count};
    MSHADOW_HIP_CALL(mshadow_hip_launch(
        reinterpret_cast<const void *>(hip::SortKeyWordKernel<KDType, false>), grid, block_dim, args,
        0, stream));
  }
  MSHADOW_HIP_CALL(mshadow_hip_sort_by_key_32(words, MSHADOW_HIP_KEY_U32, perm, n, is_ascend ? 1 : 0,
                                              base + sort_at, sort_bytes, stream));
  if (sizeof(KDType) > 4) {  // then, stably, by the high word of the keys in their new order
    void *args[] = {&words, &perm, &key_src, &cur_perm, &count};
    MSHADOW_HIP_CALL(mshadow_hip_launch(
        reinterpret_cast<const void *>(hip::SortKeyWordKernel<KDType, true>), grid, block_dim, args, 0,
        stream));
    MSHADOW_HIP_CALL(mshadow_hip_sort_by_key_32(words, MSHADOW_HIP_KEY_U32, perm, n,
                                                is_ascend ? 1 : 0, base + sort_at, sort_bytes,
                                                stream));
  }
  MSHADOW_HIP_CALL(mshadow_hip_memcpy2d_async(keys_copy, n * sizeof(KDType), keys.dptr_,
                                              n * sizeof(KDType), n * sizeof(KDType), 1,
                                              MSHADOW_HIP_D2D, stream));
  MSHADOW_HIP_CALL(mshadow_hip_memcpy2d_async(vals_copy, n * sizeof(VDType), values.dptr_,
                                              n * sizeof(VDType), n * sizeof(VDType), 1,
                                              MSHADOW_HIP_D2D, stream));
  {
    KDType *out = keys.dptr_;
    const KDType *in = keys_copy;
    void *args[] = {&out, &in, &cur_perm, &count};
    MSHADOW_HIP_CALL(mshadow_hip_launch(reinterpret_cast<const void *>(hip::SortGatherKernel<KDType>),
                                        grid, block_dim, args, 0, stream));
  }
  {
    VDType *out = values.dptr_;
    const VDType *in = vals_copy;
    void *args[] = {&out, &in, &cur_perm, &count};
    MSHADOW_HIP_CALL(mshadow_hip_launch(reinterpret_cast<const void *>(hip::SortGatherKernel<VDType>),
                                        grid, block_dim, args, 0, stream));
  }
  MSHADOW_HIP_CALL(mshadow_hip_stream_sync(stream));
  block.Release();
#else
  LOG(FATAL) << "SortByKey<gpu> of these element types: compile the calling translation unit with hipcc";
#endif
}
/*! \brief 32-bit float / integer keys with 32-bit values go to the library as they are */
template <typename KDType, typename VDType,
          bool DIRECT = (SortKeyKind<KDType>::value >= 0 && sizeof(VDType) == 4)>
struct SortRoute {
  inline static void Run(Tensor<gpu, 1, KDType> keys, Tensor<gpu, 1, VDType> values, bool is_ascend) {
    SortByKeyThroughPermutation(keys, values, is_ascend);
  }
};
template <typename KDType, typename VDType>
struct SortRoute<KDType, VDType, true> {
  inline static void Run(Tensor<gpu, 1, KDType> keys, Tensor<gpu, 1, VDType> values, bool is_ascend) {
    const size_t n = keys.size(0);
    void *stream = Stream<gpu>::GetStream(keys.stream_);
    size_t bytes = 0;
    ScopedDeviceBlock workspace;
    MSHADOW_HIP_CALL(mshadow_hip_sort_by_key_workspace(n, &bytes));
    workspace.Allocate(bytes);
    MSHADOW_HIP_CALL(mshadow_hip_sort_by_key_32(keys.dptr_, SortKeyKind<KDType>::value, values.dptr_, n,
                                                is_ascend ? 1 : 0, workspace.ptr, bytes, stream));
    MSHADOW_HIP_CALL(mshadow_hip_stream_sync(stream));
    workspace.Release();
  }
};
template <typename VDType>
struct SortRoute<half::half_t, VDType, false> {
  inline static void Run(Tensor<gpu, 1, half::half_t>, Tensor<gpu, 1, VDType>, bool) {
    LOG(FATAL) << "SortByKey is not supported for half_t keys";   // as in the reference
  }
};
}  // namespace gpu_detail
/*! \brief stable sort by key on the device (the reference: thrust::stable_sort_by_key,
 *  tensor_gpu-inl.cuh:784-806, which takes its scratch memory from the runtime as this does;
 *  half_t keys are as fatal here as there). Keys of any integer or floating type with any
 *  value type; 32-bit keys with 32-bit values are sorted in place by the library, everything
 *  else through a permutation. Returns once the sort has finished. */
template <typename KDType, typename VDType>
inline void SortByKey(Tensor<gpu, 1, KDType> keys, Tensor<gpu, 1, VDType> values,
                      bool is_ascend) {
  CHECK_EQ(keys.CheckContiguous(), true);
  CHECK_EQ(values.CheckContiguous(), true);
  CHECK_EQ(keys.size(0), values.size(0))
      << "The sizes of key/value are not equal! keys_size: " << keys.size(0)
      << "values_size: " << values.size(0);
  if (keys.size(0) == 0) return;
  gpu_detail::SortRoute<KDType, VDType>::Run(keys, values, is_ascend);
}

/* ------------------------------------------------------------------ expression routing */
namespace gpu_detail {

/*! \brief FastPath<Saver, dim, DType, E>::Run(dst, exp) returns true if it queued a
 *  fixed-function kernel for the whole assignment; the primary template matches nothing */
template <typename Saver, int dim, typename DType, typename E>
struct FastPath {
  inline static bool Run(Tensor<gpu, dim, DType> *dst, const E &exp) { return false; }
};
/* a chainer node reaches the engine as its MakeTensorExp base: match on the concrete node */
template <typename Saver, int dim, typename DType, typename Node, typename SrcExp>
struct FastPath<Saver, dim, DType, expr::MakeTensorExp<Node, SrcExp, dim, DType> > {
  inline static bool Run(Tensor<gpu, dim, DType> *dst,
                         const expr::MakeTensorExp<Node, SrcExp, dim, DType> &exp) {
    return FastPath<Saver, dim, DType, Node>::Run(dst, exp.real_self());
  }
};

/* dst = pool<Reducer>(float tensor, ...) */
template <typename Reducer, int dim>
struct FastPath<sv::saveto, dim, float,
                expr::PoolingExp<Reducer, Tensor<gpu, dim, float>, float, dim> > {
  typedef expr::PoolingExp<Reducer, Tensor<gpu, dim, float>, float, dim> E;
  inline static bool Run(Tensor<gpu, dim, float> *dst, const E &e) {
    if (ReducerCode<Reducer>::value < 0) return false;
    const Tensor<gpu, dim, float> &s = e.src_;
    MSHADOW_HIP_CALL(mshadow_hip_pool_f32(
        dst->dptr_, dst->stride_, s.dptr_, s.stride_, s.shape_.ProdShape(0, dim - 2),
        e.src_height_, e.src_width_, e.shape_[dim - 2], e.shape_[dim - 1], e.ksize_y_, e.ksize_x_,
        e.kstride_y_, e.kstride_x_, ReducerCode<Reducer>::value,
        Stream<gpu>::GetStream(dst->stream_)));
    return true;
  }
};
/* dst = unpool<Reducer>(float tensors, ...) */
template <typename Reducer, int dim>
struct FastPath<sv::saveto, dim, float,
                expr::UnPoolingExp<Reducer, Tensor<gpu, dim, float>, float, dim> > {
  typedef expr::UnPoolingExp<Reducer, Tensor<gpu, dim, float>, float, dim> E;
  inline static bool Run(Tensor<gpu, dim, float> *dst, const E &e) {
    if (ReducerCode<Reducer>::value < 0) return false;
    const Tensor<gpu, dim, float> &s = e.data_src_, &p = e.data_pooled_, &g = e.grad_pooled_;
    MSHADOW_HIP_CALL(mshadow_hip_unpool_f32(
        dst->dptr_, dst->stride_, s.dptr_, s.stride_, p.dptr_, p.stride_, g.dptr_, g.stride_,
        s.shape_.ProdShape(0, dim - 2), e.shape_[dim - 2], e.shape_[dim - 1], e.pshape_y_,
        e.pshape_x_, e.ksize_y_, e.ksize_x_, e.kstride_y_, e.kstride_x_,
        ReducerCode<Reducer>::value, Stream<gpu>::GetStream(dst->stream_)));
    return true;
  }
};

template <typename DType>
struct PatchAbi;
template <>
struct PatchAbi<float> {
  template <typename... A>
  static int Im2Col(float *col, int cs, const float *img, A... a) {
    return mshadow_hip_im2col_f32(col, cs, img, a...);
  }
  template <typename... A>
  static int Col2Im(float *img, int is, const float *col, A... a) {
    return mshadow_hip_col2im_f32(img, is, col, a...);
  }
};
template <>
struct PatchAbi<half::half_t> {
  template <typename... A>
  static int Im2Col(half::half_t *col, int cs, const half::half_t *img, A... a) {
    return mshadow_hip_im2col_f16(Bits(col), cs, Bits(img), a...);
  }
  template <typename... A>
  static int Col2Im(half::half_t *img, int is, const half::half_t *col, A... a) {
    return mshadow_hip_col2im_f16(Bits(img), is, Bits(col), a...);
  }
};
template <typename DType>
struct HasPatchAbi {
  static const bool value = false;
};
template <>
struct HasPatchAbi<float> { static const bool value = true; };
template <>
struct HasPatchAbi<half::half_t> { static const bool value = true; };

/* col = unpack_patch2col(pad(tensor, py, px), ...) and col = unpack_patch2col(tensor, ...) */
template <typename DType, int sdim>
struct FastPath<sv::saveto, 2, DType,
                expr::UnpackPatchToColXExp<
                    expr::MakeTensorExp<expr::PaddingExp<Tensor<gpu, sdim, DType>, DType, sdim>,
                                        Tensor<gpu, sdim, DType>, sdim, DType>,
                    DType, sdim> > {
  typedef expr::PaddingExp<Tensor<gpu, sdim, DType>, DType, sdim> Pad;
  typedef expr::UnpackPatchToColXExp<
      expr::MakeTensorExp<Pad, Tensor<gpu, sdim, DType>, sdim, DType>, DType, sdim> E;
  inline static bool Run(Tensor<gpu, 2, DType> *dst, const E &e) {
    if (!HasPatchAbi<DType>::value) return false;
    const Pad &p = e.img_.real_self();
    const Tensor<gpu, sdim, DType> &img = p.src_;
    MSHADOW_HIP_CALL(PatchAbi<DType>::Im2Col(
        dst->dptr_, dst->stride_, img.dptr_, img.stride_, img.shape_.ProdShape(0, sdim - 3),
        img.shape_[sdim - 3], img.shape_[sdim - 2], img.shape_[sdim - 1], e.psize_y_, e.psize_x_,
        e.pstride_y_, e.pstride_x_, e.pdilate_y_, e.pdilate_x_, p.pad_y_, p.pad_x_,
        Stream<gpu>::GetStream(dst->stream_)));
    return true;
  }
};
template <typename DType, int sdim>
struct FastPath<sv::saveto, 2, DType,
                expr::UnpackPatchToColXExp<Tensor<gpu, sdim, DType>, DType, sdim> > {
  typedef expr::UnpackPatchToColXExp<Tensor<gpu, sdim, DType>, DType, sdim> E;
  inline static bool Run(Tensor<gpu, 2, DType> *dst, const E &e) {
    if (!HasPatchAbi<DType>::value) return false;
    const Tensor<gpu, sdim, DType> &img = e.img_;
    MSHADOW_HIP_CALL(PatchAbi<DType>::Im2Col(
        dst->dptr_, dst->stride_, img.dptr_, img.stride_, img.shape_.ProdShape(0, sdim - 3),
        img.shape_[sdim - 3], img.shape_[sdim - 2], img.shape_[sdim - 1], e.psize_y_, e.psize_x_,
        e.pstride_y_, e.pstride_x_, e.pdilate_y_, e.pdilate_x_, 0, 0,
        Stream<gpu>::GetStream(dst->stream_)));
    return true;
  }
};
/* img = crop(pack_col2patch(col, padded shape, ...), (h, w), py, px) */
template <typename DType, int ddim>
struct FastPath<sv::saveto, ddim, DType,
                expr::CroppingExp<
                    expr::MakeTensorExp<expr::PackColToPatchXExp<Tensor<gpu, 2, DType>, DType, ddim>,
                                        Tensor<gpu, 2, DType>, ddim, DType>,
                    DType, ddim> > {
  typedef expr::PackColToPatchXExp<Tensor<gpu, 2, DType>, DType, ddim> Pack;
  typedef expr::CroppingExp<expr::MakeTensorExp<Pack, Tensor<gpu, 2, DType>, ddim, DType>, DType,
                            ddim> E;
  inline static bool Run(Tensor<gpu, ddim, DType> *dst, const E &e) {
    if (!HasPatchAbi<DType>::value) return false;
    const Pack &p = e.src_.real_self();
    const index_t h = e.shape_[ddim - 2], w = e.shape_[ddim - 1];
    /* the fixed-function kernel handles symmetric padding: the crop must sit pad_y / pad_x
       inside an image that is exactly 2 * pad larger */
    if (p.shape_[ddim - 2] != h + 2 * e.pad_height_ || p.shape_[ddim - 1] != w + 2 * e.pad_width_) {
      return false;
    }
    const Tensor<gpu, 2, DType> &col = p.src_;
    MSHADOW_HIP_CALL(PatchAbi<DType>::Col2Im(
        dst->dptr_, dst->stride_, col.dptr_, col.stride_, e.shape_.ProdShape(0, ddim - 3),
        e.shape_[ddim - 3], h, w, p.psize_y_, p.psize_x_, p.pstride_y_, p.pstride_x_,
        p.pdilate_y_, p.pdilate_x_, e.pad_height_, e.pad_width_,
        Stream<gpu>::GetStream(dst->stream_)));
    return true;
  }
};
/* img = pack_col2patch(col, shape, ...) without padding */
template <typename DType, int ddim>
struct FastPath<sv::saveto, ddim, DType,
                expr::PackColToPatchXExp<Tensor<gpu, 2, DType>, DType, ddim> > {
  typedef expr::PackColToPatchXExp<Tensor<gpu, 2, DType>, DType, ddim> E;
  inline static bool Run(Tensor<gpu, ddim, DType> *dst, const E &p) {
    if (!HasPatchAbi<DType>::value) return false;
    const Tensor<gpu, 2, DType> &col = p.src_;
    MSHADOW_HIP_CALL(PatchAbi<DType>::Col2Im(
        dst->dptr_, dst->stride_, col.dptr_, col.stride_, p.shape_.ProdShape(0, ddim - 3),
        p.shape_[ddim - 3], p.shape_[ddim - 2], p.shape_[ddim - 1], p.psize_y_, p.psize_x_,
        p.pstride_y_, p.pstride_x_, p.pdilate_y_, p.pdilate_x_, 0, 0,
        Stream<gpu>::GetStream(dst->stream_)));
    return true;
  }
};

/* dst = scalar (also NewTensor's initial value) on tensors of 32-bit elements */
template <int dim, typename DType>
struct FastPath<sv::saveto, dim, DType, expr::ScalarExp<DType> > {
  inline static bool Run(Tensor<gpu, dim, DType> *dst, const expr::ScalarExp<DType> &e) {
    if (sizeof(DType) != 4) return false;
    uint32_t bits = 0;
    memcpy(&bits, &e.scalar_, sizeof(DType) == 4 ? 4 : 0);
    const Shape<2> s2 = dst->shape_.FlatTo2D();
    MSHADOW_HIP_CALL(mshadow_hip_fill_32(dst->dptr_, dst->stride_, s2[0], s2[1], bits,
                                         Stream<gpu>::GetStream(dst->stream_)));
    return true;
  }
};
/* dst = transpose(tensor, axes) and dst = swapaxis<a1, a2>(tensor) on dense tensors of 32-bit
   elements: the tiled permutation of the library */
template <typename DType, int dim>
inline bool PermuteInto(Tensor<gpu, dim, DType> *dst, const Tensor<gpu, dim, DType> &src,
                        const int (&axes)[dim]) {
  if (sizeof(DType) != 4 || dim > 6 || !dst->CheckContiguous() || !src.CheckContiguous()) return false;
  int shape[dim];
  for (int i = 0; i < dim; ++i) shape[i] = static_cast<int>(src.shape_[i]);
  MSHADOW_HIP_CALL(mshadow_hip_permute_32(dst->dptr_, src.dptr_, dim, shape, axes,
                                          Stream<gpu>::GetStream(dst->stream_)));
  return true;
}
template <typename DType, int dim>
struct FastPath<sv::saveto, dim, DType, expr::TransposeExExp<Tensor<gpu, dim, DType>, DType, dim> > {
  typedef expr::TransposeExExp<Tensor<gpu, dim, DType>, DType, dim> E;
  inline static bool Run(Tensor<gpu, dim, DType> *dst, const E &e) {
    int axes[dim];
    bool seen[dim];
    for (int i = 0; i < dim; ++i) seen[i] = false;
    for (int i = 0; i < dim; ++i) {
      axes[i] = static_cast<int>(e.axes_[i]);
      if (axes[i] >= dim || seen[axes[i]]) return false;  // not a permutation: evaluated as written
      seen[axes[i]] = true;
    }
    return PermuteInto(dst, e.src_, axes);
  }
};
template <typename DType, int dim, int m_a1, int a2>
struct FastPath<sv::saveto, dim, DType,
                expr::SwapAxisExp<Tensor<gpu, dim, DType>, DType, dim, m_a1, a2> > {
  typedef expr::SwapAxisExp<Tensor<gpu, dim, DType>, DType, dim, m_a1, a2> E;
  inline static bool Run(Tensor<gpu, dim, DType> *dst, const E &e) {
    int axes[dim];
    for (int i = 0; i < dim; ++i) axes[i] = i;
    axes[dim - m_a1] = a2;
    axes[a2] = dim - m_a1;
    return PermuteInto(dst, e.src_, axes);
  }
};

/*! \brief the fixed-function routes write into plain tensors; an assignable view as the
 *  target (slice, concat, flip) always takes the generic kernel */
template <typename Saver, typename R, int dim, typename DType, typename E>
struct FastPathFor {
  inline static bool Run(R *, const E &) { return false; }
};
template <typename Saver, int dim, typename DType, typename E>
struct FastPathFor<Saver, Tensor<gpu, dim, DType>, dim, DType, E> {
  inline static bool Run(Tensor<gpu, dim, DType> *dst, const E &exp) {
    return FastPath<Saver, dim, DType, E>::Run(dst, exp);
  }
};

/*! \brief whole rows of `units` units (elements or packs) a launch of a map kernel covers:
 *  its counters are 32-bit, so fewer than 2^31 units (a margin of one workgroup's reach
 *  keeps the index of the last, partly idle, workgroup inside 32 bits) */
inline uint32_t RowsPerLaunch(uint32_t units) {
  const uint64_t limit = (1ull << 31) - (1u << 16);
  const uint64_t rows = limit / (units ? units : 1);
  return rows < 1 ? 1u : static_cast<uint32_t>(rows > 0xffffffffull ? 0xffffffffull : rows);
}

#if defined(__HIPCC__)
template <typename K>
inline void Launch(K kernel, uint32_t grid_x, uint32_t block_x, void **args, void *stream) {
  const uint32_t grid[3] = {grid_x, 1, 1};
  const uint32_t block[3] = {block_x, 1, 1};
  MSHADOW_HIP_CALL(mshadow_hip_launch(reinterpret_cast<const void *>(kernel), grid, block, args, 0,
                                      stream));
}

/*! \brief generic elementwise evaluation: pack kernel when the plan allows, else scalar */
template <typename Saver, typename DType, typename DPlan, typename SPlan, bool kPackable>
struct MapLauncher {
  inline static void Run(DPlan dplan, SPlan splan, Shape<2> shape, void *stream) {
    const uint32_t all_rows = shape[0];
    uint32_t cols = shape[1];
    if (all_rows == 0 || cols == 0) return;
    FastDivU32 div_cols(cols);
    /* the kernels count elements in 32 bits: a view of 2^31 elements or more is evaluated in
       runs of whole rows */
    const uint32_t run_rows = RowsPerLaunch(cols);
    for (uint32_t row0 = 0; row0 < all_rows; row0 += run_rows) {
      uint32_t rows = all_rows - row0 < run_rows ? all_rows - row0 : run_rows;
      uint32_t first = row0, grid = 0;
      void *args[] = {&dplan, &splan, &rows, &cols, &div_cols, &first};
      const size_t total = static_cast<size_t>(rows) * cols;
      if (cols % 4 == 0) {
        MSHADOW_HIP_CALL(mshadow_hip_suggest_grid(total / 4, hip::kMapBlock, 32, &grid));
        Launch(hip::MapScalarKernel<Saver, DType, DPlan, SPlan, 4>, grid, hip::kMapBlock, args,
               stream);
      } else {
        MSHADOW_HIP_CALL(mshadow_hip_suggest_grid(total, hip::kMapBlock, 32, &grid));
        Launch(hip::MapScalarKernel<Saver, DType, DPlan, SPlan, 1>, grid, hip::kMapBlock, args,
               stream);
      }
    }
  }
};
/*! \brief plans with a window over neighbouring planes (channel pooling) walk the planes
 *  kUnroll at a time when the rows divide into planes; false = not launched */
template <typename Saver, typename DType, int N, int kUnroll, typename DPlan, typename SPlan,
          bool kWindow>
struct PlanesLauncher {
  inline static bool Run(DPlan, SPlan, uint32_t, uint32_t, bool, void *) { return false; }
};
template <typename Saver, typename DType, int N, int kUnroll, typename DPlan, typename SPlan>
struct PlanesLauncher<Saver, DType, N, kUnroll, DPlan, SPlan, true> {
  inline static bool Run(DPlan dplan, SPlan splan, uint32_t rows, uint32_t ppr, bool stream_hint,
                         void *stream) {
    uint32_t plane_rows = static_cast<uint32_t>(splan.PlaneRows());
    if (plane_rows == 0 || rows % plane_rows != 0 || rows / plane_rows < 2) return false;
    const uint32_t planes = rows / plane_rows, plane_packs = plane_rows * ppr;
    const uint32_t places = (planes + kUnroll - 1) / kUnroll * plane_packs;
    const uint32_t grid = (places + hip::kMapBlock - 1) / hip::kMapBlock;
    uint32_t total = rows * ppr;
    FastDivU32 div_ppr(ppr), div_plane_packs(plane_packs);
    void *args[] = {&dplan, &splan, &total, &ppr, &div_ppr, &plane_rows, &div_plane_packs};
    if (stream_hint) {
      Launch(hip::MapPackPlanesKernel<Saver, DType, N, true, kUnroll, DPlan, SPlan>, grid,
             hip::kMapBlock, args, stream);
    } else {
      Launch(hip::MapPackPlanesKernel<Saver, DType, N, false, kUnroll, DPlan, SPlan>, grid,
             hip::kMapBlock, args, stream);
    }
    return true;
  }
};
template <typename Saver, typename DType, typename DPlan, typename SPlan>
struct MapLauncher<Saver, DType, DPlan, SPlan, true> {
  inline static void Run(DPlan dplan, SPlan splan, Shape<2> shape, void *stream) {
    const int N = 16 / sizeof(DType);
    uint32_t rows = shape[0], cols = shape[1];
    if (rows == 0 || cols == 0) return;
    bool flat = true;
    /* rows that are not whole packs: only for plans that evaluate a pack at any column */
    const bool ragged_ok = expr::plan_detail::RaggedRows<DPlan>::value &&
                           expr::plan_detail::RaggedRows<SPlan>::value;
    const bool aligned = (cols % N == 0 || (ragged_ok && cols >= static_cast<uint32_t>(N))) &&
                         dplan.PackReady(N, cols, &flat) && splan.PackReady(N, cols, &flat);
    if (!aligned) {
      MapLauncher<Saver, DType, DPlan, SPlan, false>::Run(dplan, splan, shape, stream);
      return;
    }
    uint32_t ppr = (cols + N - 1) / N;
    /* a plan that carries three or more tensor leaves (pointer + pitch each) is "deep" */
    const int kUnroll = sizeof(SPlan) >= 3 * (sizeof(void *) + sizeof(index_t))
                            ? hip::kPackUnrollDeep : hip::kPackUnroll;
    const uint32_t per_block = hip::kMapBlock * kUnroll;
    FastDivU32 div_ppr(ppr);
    /* streaming (non-temporal) accesses once a tensor no longer fits the caches anyway */
    const bool stream_hint = static_cast<size_t>(rows) * cols * sizeof(DType) >= (8u << 20);
    /* The kernels count packs in 32 bits, and a plan takes its column as an index_t - in a
       flat run the column is the element's offset in the whole view: a view of 2^31 ELEMENTS
       or more is evaluated in runs of whole rows (and then never as one flat run). */
    const uint32_t run_rows = RowsPerLaunch(cols);
    const bool one_run = rows <= run_rows;
    const bool is_flat = one_run && (flat || rows == 1);
    if (one_run && !is_flat && cols % N == 0 &&
        PlanesLauncher<Saver, DType, N, kUnroll, DPlan, SPlan,
                       expr::plan_detail::PlaneWindow<SPlan>::value>::Run(dplan, splan, rows, ppr,
                                                                          stream_hint, stream)) {
      return;
    }
    for (uint32_t row0 = 0; row0 < rows; row0 += run_rows) {
      uint32_t first = row0;
      const uint32_t nrows = rows - row0 < run_rows ? rows - row0 : run_rows;
      /* a flat run is one long row: only its very last pack can be partial */
      uint32_t row_elems = is_flat ? nrows * cols : cols;
      uint32_t total = is_flat ? (row_elems + N - 1) / N : nrows * ppr;
      const uint32_t grid = (total + per_block - 1) / per_block;
      void *args[] = {&dplan, &splan, &total, &ppr, &div_ppr, &first, &row_elems};
#define MSHADOW_MAP_LAUNCH(FLAT, STREAM)                                                   \
  Launch(hip::MapPackKernel<Saver, DType, N, FLAT, STREAM, kUnroll, DPlan, SPlan>, grid,   \
         hip::kMapBlock, args, stream)
      if (is_flat && stream_hint) {
        MSHADOW_MAP_LAUNCH(true, true);
      } else if (is_flat) {
        MSHADOW_MAP_LAUNCH(true, false);
      } else if (stream_hint) {
        MSHADOW_MAP_LAUNCH(false, true);
      } else {
        MSHADOW_MAP_LAUNCH(false, false);
      }
#undef MSHADOW_MAP_LAUNCH
    }
  }
};
#endif  // __HIPCC__

}  // namespace gpu_detail

template <typename Saver, typename R, int dim, typename DType, typename E, int etype>
inline void MapExp(TRValue<R, gpu, dim, DType> *dst, const expr::Exp<E, DType, etype> &exp) {
  expr::TypeCheckPass<expr::TypeCheck<gpu, dim, DType, E>::kMapPass>::
      Error_All_Tensor_in_Exp_Must_Have_Same_Type();
  Shape<dim> eshape = expr::ShapeCheck<dim, E>::Check(exp.self());
  Shape<dim> dshape = expr::ShapeCheck<dim, R>::Check(dst->self());
  CHECK(eshape[0] == 0 || eshape == dshape)
      << "Assignment: Shape of Tensors are not consistent with target, "
      << "eshape: " << eshape << " dshape:" << dshape;
  if (gpu_detail::FastPathFor<Saver, R, dim, DType, E>::Run(dst->ptrself(), exp.self())) return;
#if defined(__HIPCC__)
  typedef expr::Plan<R, DType> DPlan;
  typedef expr::Plan<E, DType> SPlan;
  gpu_detail::MapLauncher<Saver, DType, DPlan, SPlan,
                          expr::plan_detail::Packable<DPlan>::value &&
                              expr::plan_detail::Packable<SPlan>::value>::
      Run(expr::MakePlan(dst->self()), expr::MakePlan(exp.self()), dshape.FlatTo2D(),
          Stream<gpu>::GetStream(expr::StreamInfo<gpu, R>::Get(dst->self())));
#else
  LOG(FATAL) << "MapExp<gpu>: this expression has no fixed-function kernel; compile the "
                "calling translation unit with hipcc so that its kernel can be instantiated";
#endif
}

namespace gpu_detail {
/*! \brief reductions whose source is a float tensor in memory and whose reducer / saver are
 *  the built-in ones go to the fixed-function entry points of the library, which fetch
 *  the tensor straight into LDS; every other reduction (an expression source, another
 *  element type, a caller-defined reducer) is compiled from the generic kernel templates */
template <typename Saver, typename Reducer, typename R, typename E, typename DType>
struct ReduceRoute {
  static const bool kFixed = false;
  template <typename... Args> static void Lowest(Args...) {}
  template <typename... Args> static void HighDim(Args...) {}
};
template <typename Saver, typename Reducer, int dim>
struct ReduceRoute<Saver, Reducer, Tensor<gpu, 1, float>, Tensor<gpu, dim, float>, float> {
  static const bool kFixed = SaverCode<Saver>::value >= 0 && ReducerCode<Reducer>::value >= 0;
  static void Lowest(const Tensor<gpu, 1, float> &dst, const Tensor<gpu, dim, float> &src,
                     uint32_t rows, uint32_t cols, float scale) {
    MSHADOW_HIP_CALL(mshadow_hip_reduce_keep_lowest_f32(
        dst.dptr_, src.dptr_, static_cast<int>(src.stride_), static_cast<int>(rows),
        static_cast<int>(cols), ReducerCode<Reducer>::value, SaverCode<Saver>::value, scale,
        Stream<gpu>::GetStream(dst.stream_)));
  }
  static void HighDim(const Tensor<gpu, 1, float> &dst, const Tensor<gpu, dim, float> &src,
                      uint32_t n_out, uint32_t n_keep, uint32_t n_y, uint32_t n_x, float scale) {
    MSHADOW_HIP_CALL(mshadow_hip_reduce_keep_highdim_f32(
        dst.dptr_, src.dptr_, static_cast<int>(src.stride_), static_cast<int>(n_out),
        static_cast<int>(n_keep), static_cast<int>(n_y), static_cast<int>(n_x),
        ReducerCode<Reducer>::value, SaverCode<Saver>::value, scale,
        Stream<gpu>::GetStream(dst.stream_)));
  }
};
#if defined(__HIPCC__)
/*! \brief sumall_except_dim of a half_t tensor in memory: the LDS-ring kernel of the float path
 *  (kernels/reduce_dma.h) instantiated for 16-bit elements, a load bringing two neighbouring
 *  elements of a row. Run() returns false when the shape does not allow that (odd row length or
 *  pitch, unaligned base, little work per kept index) and the generic kernel has to do it. */
template <typename Saver, typename Reducer, typename R, typename E>
struct HalfRingRoute {
  template <typename... Args> static bool HighDim(Args...) { return false; }
};
template <typename Saver, typename Reducer, int dim>
struct HalfRingRoute<Saver, Reducer, Tensor<gpu, 1, half::half_t>, Tensor<gpu, dim, half::half_t> > {
  static bool HighDim(const Tensor<gpu, 1, half::half_t> &dst, const Tensor<gpu, dim, half::half_t> &src,
                      uint32_t n_out, uint32_t n_keep, uint32_t n_y, uint32_t n_x,
                      half::half_t scale) {
    const uint64_t per_kept = static_cast<uint64_t>(n_out) * n_y * n_x;
    if (n_x % 2 != 0 || src.stride_ % 2 != 0 || reinterpret_cast<uintptr_t>(src.dptr_) % 4 != 0 ||
        per_kept < (1u << 16) || static_cast<uint64_t>(n_y) * n_x >= (1ull << 31)) {
      return false;
    }
    half::half_t *d = dst.dptr_;
    const half::half_t *s = src.dptr_;
    uint32_t stride = src.stride_;
    void *stream = Stream<gpu>::GetStream(dst.stream_);
    /* the inner chains spread over as many workgroups as there are groups of segments, where
       rows are whole 16-byte packs (dense rows are walked as one row per segment) and the
       library has scratch memory for the inner results of this stream */
    {
      uint32_t v_y = n_y, v_x = n_x, v_stride = stride;
      if (stride == n_x) {
        v_x = v_stride = n_y * n_x;
        v_y = 1;
      }
      uint32_t *partial = NULL, *counter = NULL;
      /* fewer kept indices than CUs (the chip's 256: the one-workgroup-per-kept-index kernel
         below would leave some idle): the inner chains are dealt out by segments */
      const bool few_kept = n_keep < 192u;
      const bool packs = v_x % 8 == 0 && v_stride % 8 == 0 && reinterpret_cast<uintptr_t>(s) % 16 == 0;
      if (few_kept && static_cast<uint64_t>(n_out) * n_keep < (1ull << 31)) {
        MSHADOW_HIP_CALL(mshadow_hip_reduce_scratch(stream, static_cast<size_t>(n_out) * n_keep,
                                                    &partial, &counter));
      }
      if (partial != NULL) {
        FastDivU32 v_div_x(v_x);
        void *sargs[] = {&d, &s, &v_stride, &n_out, &n_keep, &v_y, &v_x, &v_div_x, &scale, &partial,
                         &counter};
        if (packs) {
          typedef hip::HighDimSplitRingPacks Ring;
          Launch(hip::ReduceKeepHighDimSplitKernel<Saver, Reducer, half::half_t, Ring>,
                 (n_out * n_keep + Ring::kSegs - 1) / Ring::kSegs, Ring::kThreads, sargs, stream);
        } else {
          typedef hip::HighDimSplitRing Ring;
          Launch(hip::ReduceKeepHighDimSplitKernel<Saver, Reducer, half::half_t, Ring>,
                 (n_out * n_keep + Ring::kSegs - 1) / Ring::kSegs, Ring::kThreads, sargs, stream);
        }
        return true;
      }
    }
    FastDivU32 div_x(n_x);
    void *args[] = {&d, &s, &stride, &n_out, &n_keep, &n_y, &n_x, &div_x, &scale};
#define MSHADOW_HALF_RING(SEGS)                                                                  \
    Launch(hip::ReduceKeepHighDimDmaKernel<Saver, Reducer, half::half_t, SEGS>, n_keep,         \
           hip::kDmaThreads, args, stream)
    if (n_out > 16) MSHADOW_HALF_RING(64);
    else if (n_out > 4) MSHADOW_HALF_RING(16);
    else if (n_out > 1) MSHADOW_HALF_RING(4);
    else MSHADOW_HALF_RING(1);
#undef MSHADOW_HALF_RING
    return true;
  }
};
#endif  // __HIPCC__
}  // namespace gpu_detail

template <typename Saver, typename Reducer, typename R, typename DType, typename E, int etype>
inline void MapReduceKeepLowest(TRValue<R, gpu, 1, DType> *dst,
                                const expr::Exp<E, DType, etype> &exp, DType scale) {
  expr::TypeCheckPass<expr::TypeCheck<gpu, 1, DType, E>::kRedPass>::
      Error_TypeCheck_Not_Pass_For_Reduce_Exp();
  Shape<2> eshape = expr::ShapeCheck<expr::ExpInfo<E>::kDim, E>::Check(exp.self()).FlatTo2D();
  Shape<1> dshape = expr::ShapeCheck<1, R>::Check(dst->self());
  CHECK_EQ(eshape[1], dshape[0]) << "MapReduceKeepLowest::reduction dimension do not match";
  CHECK_NE(eshape[0], 0U) << "can not reduce over empty tensor";
  typedef gpu_detail::ReduceRoute<Saver, Reducer, R, E, DType> Route;
  if (Route::kFixed) {
    Route::Lowest(dst->self(), exp.self(), eshape[0], eshape[1], scale);
    return;
  }
#if defined(__HIPCC__)
  typedef expr::Plan<R, DType> DPlan;
  typedef expr::Plan<E, DType> SPlan;
  DPlan dplan = expr::MakePlan(dst->self());
  SPlan splan = expr::MakePlan(exp.self());
  uint32_t rows = eshape[0], cols = eshape[1];
  if (cols == 0) return;
  void *args[] = {&dplan, &splan, &rows, &cols, &scale};
  void *stream = Stream<gpu>::GetStream(expr::StreamInfo<gpu, R>::Get(dst->self()));
  const uint32_t strips = (cols + hip::kLowestCols - 1) / hip::kLowestCols;
  if (rows >= 4096) {
    gpu_detail::Launch(hip::ReduceKeepLowestKernel<Saver, Reducer, DType, hip::RedBlockLargeFor<DType>::value,
                                                   DPlan, SPlan>,
                       strips, hip::RedBlockLargeFor<DType>::value, args, stream);
  } else {
    gpu_detail::Launch(hip::ReduceKeepLowestKernel<Saver, Reducer, DType, hip::kRedBlockSmall,
                                                   DPlan, SPlan>,
                       strips, hip::kRedBlockSmall, args, stream);
  }
#else
  LOG(FATAL) << "MapReduceKeepLowest<gpu>: compile the calling translation unit with hipcc";
#endif
}

template <typename Saver, typename Reducer, int dimkeep, typename R, typename DType, typename E,
          int etype>
inline void MapReduceKeepHighDim(TRValue<R, gpu, 1, DType> *dst,
                                 const expr::Exp<E, DType, etype> &exp, DType scale) {
  expr::TypeCheckPass<expr::TypeCheck<gpu, dimkeep, DType, E>::kRedPass>::
      Error_TypeCheck_Not_Pass_For_Reduce_Exp();
  typedef Shape<expr::ExpInfo<E>::kDim> EShape;
  EShape eshape = expr::ShapeCheck<expr::ExpInfo<E>::kDim, E>::Check(exp.self());
  Shape<1> dshape = expr::ShapeCheck<1, R>::Check(dst->self());
  CHECK_EQ(eshape[dimkeep], dshape[0]) << "MapReduceKeepHighDim::reduction dimension do not match";
  typedef gpu_detail::ReduceRoute<Saver, Reducer, R, E, DType> Route;
  if (Route::kFixed) {
    Route::HighDim(dst->self(), exp.self(), eshape.ProdShape(0, dimkeep), eshape[dimkeep],
                   eshape.ProdShape(dimkeep + 1, EShape::kSubdim), eshape[EShape::kSubdim], scale);
    return;
  }
#if defined(__HIPCC__)
  typedef expr::Plan<R, DType> DPlan;
  typedef expr::Plan<E, DType> SPlan;
  DPlan dplan = expr::MakePlan(dst->self());
  SPlan splan = expr::MakePlan(exp.self());
  uint32_t n_out = eshape.ProdShape(0, dimkeep), n_keep = eshape[dimkeep];
  uint32_t n_y = eshape.ProdShape(dimkeep + 1, EShape::kSubdim), n_x = eshape[EShape::kSubdim];
  if (n_keep == 0) return;
  if (n_out > 0 && n_y > 0 && n_x > 0 &&
      gpu_detail::HalfRingRoute<Saver, Reducer, R, E>::HighDim(dst->self(), exp.self(), n_out, n_keep,
                                                               n_y, n_x, scale)) {
    return;
  }
  CHECK_LT(static_cast<uint64_t>(n_y) * n_x, 1ull << 31) << "MapReduceKeepHighDim: inner extent too large";
  FastDivU32 div_x(n_x > 0 ? n_x : 1);
  void *args[] = {&dplan, &splan, &n_out, &n_keep, &n_y, &n_x, &div_x, &scale};
  void *stream = Stream<gpu>::GetStream(expr::StreamInfo<gpu, R>::Get(dst->self()));
  /* segments staged side by side = chain lanes in use (fewer, longer pieces when the
     outer extent is small); the large workgroup when each kept index has enough work */
  const bool large = static_cast<uint64_t>(n_out) * n_y * n_x >= (1u << 18);
#define MSHADOW_HIGHDIM_LAUNCH(SEGS)                                                          \
  if (large) {                                                                                \
    gpu_detail::Launch(hip::ReduceKeepHighDimKernel<Saver, Reducer, DType, hip::RedBlockLargeFor<DType>::value, \
                                                    SEGS, DPlan, SPlan>,                      \
                       n_keep, hip::RedBlockLargeFor<DType>::value, args, stream);                            \
  } else {                                                                                    \
    gpu_detail::Launch(hip::ReduceKeepHighDimKernel<Saver, Reducer, DType, hip::kRedBlockSmall, \
                                                    SEGS, DPlan, SPlan>,                      \
                       n_keep, hip::kRedBlockSmall, args, stream);                            \
  }
  if (n_out > 16) {
    MSHADOW_HIGHDIM_LAUNCH(64)
  } else if (n_out > 4) {
    MSHADOW_HIGHDIM_LAUNCH(16)
  } else if (n_out > 1) {
    MSHADOW_HIGHDIM_LAUNCH(4)
  } else {
    MSHADOW_HIGHDIM_LAUNCH(1)
  }
#undef MSHADOW_HIGHDIM_LAUNCH
#else
  LOG(FATAL) << "MapReduceKeepHighDim<gpu>: compile the calling translation unit with hipcc";
#endif
}

}  // namespace mshadow
#endif  // MSHADOW_HIP_TENSOR_GPU_H_
