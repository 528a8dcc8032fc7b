/*
 * SaveBinary / LoadBinary: a tensor as a flat binary record.
 *
 * The record is what mshadow/io.h:88-133 of the reference writes: the Shape<dim> object
 * (dim index_t values), then the elements row by row without the pitch padding. Any stream
 * type with `size_t Read(void*, size_t)` and `void Write(const void*, size_t)` serves
 * (utils::IStream is the abstract form). Tensors on the GPU pass through a host copy.
 * LoadBinary with pre_alloc = false allocates *dst (the caller frees it); with pre_alloc =
 * true the stored shape must equal dst's.
 */
#ifndef MSHADOW_IO_H_
#define MSHADOW_IO_H_

#include "./tensor.h"

namespace mshadow {
namespace utils {
/*! \brief the stream interface SaveBinary / LoadBinary need */
class IStream {
 public:
  /*! \brief read up to size bytes; returns the number of bytes read (0 at the end) */
  virtual size_t Read(void *ptr, size_t size) = 0;
  virtual void Write(const void *ptr, size_t size) = 0;
  virtual ~IStream(void) {}
};
}  // namespace utils

template <int dim, typename DType, typename TStream>
inline void SaveBinary(TStream &fo, const Tensor<cpu, dim, DType> &src) {  // NOLINT(*)
  fo.Write(&src.shape_, sizeof(src.shape_));
  const Tensor<cpu, 2, DType> rows = src.FlatTo2D();
  for (index_t y = 0; y < rows.size(0); ++y) fo.Write(rows[y].dptr_, sizeof(DType) * rows.size(1));
}

template <int dim, typename DType, typename TStream>
inline void LoadBinary(TStream &fi, Tensor<cpu, dim, DType> *dst, bool pre_alloc) {  // NOLINT(*)
  Shape<dim> shape;
  CHECK_NE(fi.Read(&shape, sizeof(shape)), 0U) << "mshadow::LoadBinary";
  if (pre_alloc) {
    CHECK_EQ(shape, dst->shape_) << "LoadBinary, shape do not match pre-allocated shape";
  } else {
    dst->shape_ = shape;
    AllocSpace(dst);
  }
  Tensor<cpu, 2, DType> rows = dst->FlatTo2D();
  for (index_t y = 0; y < rows.size(0); ++y) {
    if (rows.size(1) == 0) break;
    CHECK_NE(fi.Read(rows[y].dptr_, sizeof(DType) * rows.size(1)), 0U) << "mshadow::LoadBinary";
  }
}

/* device tensors: through a dense host copy; the calls return when the copy has finished */
template <int dim, typename DType, typename TStream>
inline void SaveBinary(TStream &fo, const Tensor<gpu, dim, DType> &src) {  // NOLINT(*)
  Tensor<cpu, dim, DType> host(src.shape_);
  AllocSpace(&host, false);
  Copy(host, src, src.stream_);
  if (src.stream_ != NULL) src.stream_->Wait();
  SaveBinary(fo, host);
  FreeSpace(&host);
}

template <int dim, typename DType, typename TStream>
inline void LoadBinary(TStream &fi, Tensor<gpu, dim, DType> *dst, bool pre_alloc) {  // NOLINT(*)
  Tensor<cpu, dim, DType> host;
  LoadBinary(fi, &host, false);
  if (pre_alloc) {
    CHECK_EQ(host.shape_, dst->shape_) << "LoadBinary, shape do not match pre-allocated shape";
  } else {
    dst->shape_ = host.shape_;
    AllocSpace(dst);
  }
  Copy(*dst, host, dst->stream_);
  if (dst->stream_ != NULL) dst->stream_->Wait();
  FreeSpace(&host);
}

}  // namespace mshadow
#endif  // MSHADOW_IO_H_
