/*
 * Shape<N>: dimension sizes of a tensor, highest dimension first (numpy order).
 * Interface per mshadow/tensor.h:50-242 of the reference; every N-d tensor is
 * evaluated as the 2-D matrix FlatTo2D() = (product of leading dims, last dim).
 */
#ifndef MSHADOW_CORE_SHAPE_H_
#define MSHADOW_CORE_SHAPE_H_

#include <iostream>

#include "../base.h"

namespace mshadow {

template <int dimension>
struct Shape {
  static const int kDimension = dimension;
  static const int kSubdim = dimension - 1;
  index_t shape_[kDimension];

  MSHADOW_XINLINE Shape(void) {}
  MSHADOW_XINLINE Shape(const Shape<kDimension> &s) {
#pragma unroll
    for (int i = 0; i < kDimension; ++i) shape_[i] = s.shape_[i];
  }
  MSHADOW_XINLINE Shape<kDimension> &operator=(const Shape<kDimension> &s) {
#pragma unroll
    for (int i = 0; i < kDimension; ++i) shape_[i] = s.shape_[i];
    return *this;
  }
  MSHADOW_XINLINE index_t &operator[](index_t idx) { return shape_[idx]; }
  MSHADOW_XINLINE const index_t &operator[](index_t idx) const { return shape_[idx]; }
  MSHADOW_XINLINE bool operator==(const Shape<kDimension> &s) const {
    bool same = true;
#pragma unroll
    for (int i = 0; i < kDimension; ++i) same = same && (s.shape_[i] == shape_[i]);
    return same;
  }
  MSHADOW_XINLINE bool operator!=(const Shape<kDimension> &s) const { return !(*this == s); }
  /*! \brief product of the sizes in [dimstart, dimend) */
  MSHADOW_XINLINE index_t ProdShape(int dimstart, int dimend) const {
    index_t num = 1;
#pragma unroll
    for (int i = dimstart; i < dimend; ++i) num *= shape_[i];
    return num;
  }
  /*! \brief number of elements */
  MSHADOW_XINLINE index_t Size(void) const { return ProdShape(0, kDimension); }
  MSHADOW_XINLINE Shape<1> FlatTo1D(void) const {
    Shape<1> s;
    s[0] = Size();
    return s;
  }
  /*! \brief (product of all but the last dimension, last dimension) */
  MSHADOW_XINLINE Shape<2> FlatTo2D(void) const {
    Shape<2> s;
    s.shape_[0] = ProdShape(0, kDimension - 1);
    s.shape_[1] = shape_[kDimension - 1];
    return s;
  }
  /*! \brief drop the highest dimension */
  MSHADOW_XINLINE Shape<kSubdim> SubShape(void) const {
    Shape<kSubdim> s;
#pragma unroll
    for (int i = 0; i < kSubdim; ++i) s.shape_[i] = shape_[i + 1];
    return s;
  }
  /*! \brief dimensions [dimstart, dimend) as a shape of their own */
  template <int dimstart, int dimend>
  MSHADOW_XINLINE Shape<dimend - dimstart> Slice(void) const {
    Shape<dimend - dimstart> s;
#pragma unroll
    for (int i = dimstart; i < dimend; ++i) s[i - dimstart] = shape_[i];
    return s;
  }
};

MSHADOW_XINLINE Shape<1> Shape1(index_t s0) {
  Shape<1> s;
  s[0] = s0;
  return s;
}
MSHADOW_XINLINE Shape<2> Shape2(index_t s0, index_t s1) {
  Shape<2> s;
  s[0] = s0; s[1] = s1;
  return s;
}
MSHADOW_XINLINE Shape<3> Shape3(index_t s0, index_t s1, index_t s2) {
  Shape<3> s;
  s[0] = s0; s[1] = s1; s[2] = s2;
  return s;
}
MSHADOW_XINLINE Shape<4> Shape4(index_t s0, index_t s1, index_t s2, index_t s3) {
  Shape<4> s;
  s[0] = s0; s[1] = s1; s[2] = s2; s[3] = s3;
  return s;
}
MSHADOW_XINLINE Shape<5> Shape5(index_t s0, index_t s1, index_t s2, index_t s3, index_t s4) {
  Shape<5> s;
  s[0] = s0; s[1] = s1; s[2] = s2; s[3] = s3; s[4] = s4;
  return s;
}

/*! \brief python-tuple style printing: (2,3) and (5,) - mshadow/tensor_cpu-inl.h:40-51 */
template <int ndim>
inline std::ostream &operator<<(std::ostream &os, const Shape<ndim> &shape) {  // NOLINT(*)
  os << '(';
  for (int i = 0; i < ndim; ++i) {
    if (i != 0) os << ',';
    os << shape[i];
  }
  if (ndim == 1) os << ',';
  os << ')';
  return os;
}

namespace layout_detail {
/* position of each logical axis (N, C, spatial...) inside a stored layout */
template <int ndim>
inline bool AxisOrder(int layout, int *perm);
template <>
inline bool AxisOrder<3>(int layout, int *perm) {  // logical (N, C, W)
  if (layout == kNCW) { perm[0] = 0; perm[1] = 1; perm[2] = 2; return true; }
  if (layout == kNWC) { perm[0] = 0; perm[1] = 2; perm[2] = 1; return true; }
  return false;
}
template <>
inline bool AxisOrder<4>(int layout, int *perm) {  // logical (N, C, H, W)
  if (layout == kNCHW) { perm[0] = 0; perm[1] = 1; perm[2] = 2; perm[3] = 3; return true; }
  if (layout == kNHWC) { perm[0] = 0; perm[1] = 3; perm[2] = 1; perm[3] = 2; return true; }
  return false;
}
template <>
inline bool AxisOrder<5>(int layout, int *perm) {  // logical (N, C, D, H, W)
  if (layout == kNCDHW) { perm[0] = 0; perm[1] = 1; perm[2] = 2; perm[3] = 3; perm[4] = 4; return true; }
  if (layout == kNDHWC) { perm[0] = 0; perm[1] = 4; perm[2] = 1; perm[3] = 2; perm[4] = 3; return true; }
  return false;
}
template <int ndim>
inline Shape<ndim> Convert(const Shape<ndim> &src, int src_layout, int dst_layout) {
  int from[ndim], to[ndim];
  if (!AxisOrder<ndim>(src_layout, from)) {
    LOG(FATAL) << "Invalid layout for " << ndim << "d shape " << src_layout;
  }
  if (!AxisOrder<ndim>(dst_layout, to)) {
    LOG(FATAL) << "Invalid layout for " << ndim << "d shape " << dst_layout;
  }
  Shape<ndim> logical, dst;
  for (int i = 0; i < ndim; ++i) logical[i] = src[from[i]];
  for (int i = 0; i < ndim; ++i) dst[to[i]] = logical[i];
  return dst;
}
}  // namespace layout_detail

/*! \brief re-express a shape stored in src_layout in dst_layout (mshadow/tensor.h:251-359) */
inline Shape<3> ConvertLayout(const Shape<3> &src, int src_layout, int dst_layout) {
  return layout_detail::Convert<3>(src, src_layout, dst_layout);
}
inline Shape<4> ConvertLayout(const Shape<4> &src, int src_layout, int dst_layout) {
  return layout_detail::Convert<4>(src, src_layout, dst_layout);
}
inline Shape<5> ConvertLayout(const Shape<5> &src, int src_layout, int dst_layout) {
  return layout_detail::Convert<5>(src, src_layout, dst_layout);
}

}  // namespace mshadow
#endif  // MSHADOW_CORE_SHAPE_H_
