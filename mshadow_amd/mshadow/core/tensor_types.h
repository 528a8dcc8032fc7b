/*
 * Device tags, Stream<Device> and the Tensor handle.
 *
 * A Tensor is a plain handle {dptr_, shape_, stride_, stream_}: copying it copies the
 * handle, never the data, and memory is always allocated and freed explicitly.
 * stride_ is the row pitch of the 2-D view in elements. Member names and constructor
 * forms follow mshadow/tensor.h:21-33 and :364-614 of the reference.
 */
#ifndef MSHADOW_CORE_TENSOR_TYPES_H_
#define MSHADOW_CORE_TENSOR_TYPES_H_

#include "../expr/nodes.h"
#include "./shape.h"

namespace mshadow {

/*! \brief device name CPU */
struct cpu {
  static const bool kDevCPU = true;
  static const int kDevMask = 1 << 0;
};
/*! \brief device name GPU (one gfx950 device) */
struct gpu {
  static const bool kDevCPU = false;
  static const int kDevMask = 1 << 1;
};

/*! \brief computation stream; the CPU one is a no-op, Stream<gpu> is specialised */
template <typename Device>
struct Stream {
  inline void Wait(void) {}
  inline bool CheckIdle(void) { return true; }
  inline void CreateBlasHandle() {}
};

/*! \brief super type of everything that owns elements on a device */
template <typename Container, typename Device, int dimension, typename DType>
struct TRValue : public expr::RValueExp<Container, DType> {};

template <typename Device, int dimension, typename DType MSHADOW_DEFAULT_DTYPE>
struct Tensor : public TRValue<Tensor<Device, dimension, DType>, Device, dimension, DType> {
 public:
  static const bool kDevCPU = Device::kDevCPU;
  static const int kSubdim = dimension - 1;
  /*! \brief pointer to the data */
  DType *dptr_ = nullptr;
  /*! \brief shape of the tensor */
  Shape<dimension> shape_;
  /*! \brief row pitch in elements (>= shape_[dimension-1]) */
  index_t stride_;
  /*! \brief stream the computation on this tensor is queued to */
  Stream<Device> *stream_;

  MSHADOW_XINLINE Tensor(void) : stream_(NULL) {}
  MSHADOW_XINLINE Tensor(const Shape<dimension> &shape) : shape_(shape), stream_(NULL) {}  // NOLINT(*)
  MSHADOW_XINLINE Tensor(DType *dptr, const Shape<dimension> &shape)
      : dptr_(dptr), shape_(shape), stride_(shape[kSubdim]), stream_(NULL) {}
  MSHADOW_XINLINE Tensor(DType *dptr, const Shape<dimension> &shape, Stream<Device> *stream)
      : dptr_(dptr), shape_(shape), stride_(shape[kSubdim]), stream_(stream) {}
  MSHADOW_XINLINE Tensor(DType *dptr, const Shape<dimension> &shape, index_t stride,
                         Stream<Device> *stream)
      : dptr_(dptr), shape_(shape), stride_(stride), stream_(stream) {}

  inline void set_stream(Stream<Device> *stream) { this->stream_ = stream; }
  /*! \brief elements spanned by dimensions startdim.., counting the padded pitch */
  template <int startdim>
  MSHADOW_XINLINE index_t MemSize(void) const {
    index_t memsz = this->stride_;
#pragma unroll
    for (int i = startdim; i < kSubdim; ++i) memsz *= this->shape_[i];
    return memsz;
  }
  MSHADOW_XINLINE bool CheckContiguous(void) const { return this->shape_[dimension - 1] == stride_; }
  MSHADOW_XINLINE index_t MSize(void) const { return this->MemSize<0>(); }
  MSHADOW_XINLINE index_t size(index_t idx) const { return shape_[idx]; }
  MSHADOW_XINLINE Tensor<Device, 1, DType> FlatTo1D(void) const {
    return Tensor<Device, 1, DType>(dptr_, shape_.FlatTo1D(), stride_, stream_);
  }
  MSHADOW_XINLINE Tensor<Device, 2, DType> FlatTo2D(void) const {
    return Tensor<Device, 2, DType>(dptr_, shape_.FlatTo2D(), stride_, stream_);
  }
  /*! \brief sub-tensor idx of the highest dimension */
  MSHADOW_XINLINE Tensor<Device, kSubdim, DType> operator[](index_t idx) const {
    return Tensor<Device, kSubdim, DType>(dptr_ + this->MemSize<1>() * idx, shape_.SubShape(),
                                          stride_, stream_);
  }
  /*! \brief [begin, end) of the highest dimension */
  MSHADOW_XINLINE Tensor<Device, dimension, DType> Slice(index_t begin, index_t end) const {
    Shape<dimension> s = this->shape_;
    s[0] = end - begin;
    return Tensor<Device, dimension, DType>(dptr_ + this->MemSize<1>() * begin, s, stride_, stream_);
  }
  /*! \brief handle assignment */
  inline Tensor<Device, dimension, DType> &operator=(const Tensor<Device, dimension, DType> &exp) {
    dptr_ = exp.dptr_;
    shape_ = exp.shape_;
    stride_ = exp.stride_;
    stream_ = exp.stream_;
    return *this;
  }
  /*! \brief evaluate an expression into this tensor */
  template <typename E, int etype>
  inline Tensor<Device, dimension, DType> &operator=(const expr::Exp<E, DType, etype> &exp) {
    return this->__assign(exp);
  }
  inline Tensor<Device, dimension, DType> &operator=(const DType &exp) { return this->__assign(exp); }
};

/*! \brief 1-D tensors index to elements, not sub-tensors (mshadow/tensor.h:549-614) */
template <typename Device, typename DType>
struct Tensor<Device, 1, DType> : public TRValue<Tensor<Device, 1, DType>, Device, 1, DType> {
 public:
  DType *dptr_;
  Shape<1> shape_;
  index_t stride_;
  Stream<Device> *stream_;

  MSHADOW_XINLINE Tensor(void) : stream_(NULL) {}
  MSHADOW_XINLINE Tensor(const Shape<1> &shape) : shape_(shape), stream_(NULL) {}  // NOLINT(*)
  MSHADOW_XINLINE Tensor(DType *dptr, Shape<1> shape)
      : dptr_(dptr), shape_(shape), stride_(shape[0]), stream_(NULL) {}
  MSHADOW_XINLINE Tensor(DType *dptr, Shape<1> shape, Stream<Device> *stream)
      : dptr_(dptr), shape_(shape), stride_(shape[0]), stream_(stream) {}
  MSHADOW_XINLINE Tensor(DType *dptr, Shape<1> shape, index_t stride, Stream<Device> *stream)
      : dptr_(dptr), shape_(shape), stride_(stride), stream_(stream) {}

  inline void set_stream(Stream<Device> *stream) { this->stream_ = stream; }
  MSHADOW_XINLINE Tensor<Device, 1, DType> FlatTo1D(void) const { return *this; }
  MSHADOW_XINLINE Tensor<Device, 2, DType> FlatTo2D(void) const {
    return Tensor<Device, 2, DType>(dptr_, shape_.FlatTo2D(), stride_, stream_);
  }
  MSHADOW_XINLINE Tensor<Device, 1, DType> Slice(index_t begin, index_t end) const {
    Shape<1> s;
    s[0] = end - begin;
    return Tensor<Device, 1, DType>(dptr_ + begin, s, s[0], stream_);
  }
  MSHADOW_XINLINE bool CheckContiguous(void) const { return true; }
  MSHADOW_XINLINE index_t MSize(void) const { return shape_[0]; }
  MSHADOW_XINLINE index_t size(index_t i) const { return shape_[0]; }
  MSHADOW_XINLINE DType &operator[](index_t idx) { return dptr_[idx]; }
  MSHADOW_XINLINE const DType &operator[](index_t idx) const { return dptr_[idx]; }
  inline Tensor<Device, 1, DType> &operator=(const Tensor<Device, 1, DType> &exp) {
    dptr_ = exp.dptr_;
    shape_ = exp.shape_;
    stride_ = exp.stride_;
    stream_ = exp.stream_;
    return *this;
  }
  template <typename E, int etype>
  inline Tensor<Device, 1, DType> &operator=(const expr::Exp<E, DType, etype> &exp) {
    return this->__assign(exp);
  }
  inline Tensor<Device, 1, DType> &operator=(const DType &exp) { return this->__assign(exp); }
};

}  // namespace mshadow
#endif  // MSHADOW_CORE_TENSOR_TYPES_H_
