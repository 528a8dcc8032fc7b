/*
 * TensorContainer: a Tensor that owns its memory. The interface is the one declared at
 * mshadow/tensor_container.h:24-205 of the reference (constructors, Resize, Release, set_pad,
 * SaveBinary / LoadBinary, the assignment forms); the bookkeeping is this file's own.
 *
 * The container holds one block of `rows x pitch` elements, obtained from AllocSpace. The
 * Tensor part of the object is a view of that block under the current shape: Resize only
 * moves the view while the requested shape fits the block (rows and row length), and takes
 * a new block otherwise - the old contents are not kept in either case. With padding the
 * view keeps the block's pitch, without it rows are dense. Copying a container copies the
 * elements; handing it to a function that takes a plain Tensor passes a non-owning view.
 */
#ifndef MSHADOW_TENSOR_CONTAINER_H_
#define MSHADOW_TENSOR_CONTAINER_H_

#include "./io.h"
#include "./tensor.h"

namespace mshadow {

template <typename Device, int dimension, typename DType = default_real_t>
class TensorContainer : public Tensor<Device, dimension, DType> {
  typedef Tensor<Device, dimension, DType> View;
  typedef Tensor<Device, 2, DType> Rows;

 public:
  /*! \brief an empty container; memory comes with the first Resize */
  explicit TensorContainer(bool pad = MSHADOW_ALLOC_PAD) : block_(NULL), rows_(0), pitch_(0), padded_(pad) {
    this->PointNowhere();
  }
  explicit TensorContainer(const Shape<dimension> &shape)
      : block_(NULL), rows_(0), pitch_(0), padded_(MSHADOW_ALLOC_PAD) {
    this->TakeBlockFor(shape);
  }
  TensorContainer(const Shape<dimension> &shape, DType initv)
      : block_(NULL), rows_(0), pitch_(0), padded_(MSHADOW_ALLOC_PAD) {
    this->TakeBlockFor(shape);
    (*this) = initv;
  }
  /*! \brief a copy of the elements (and of the padding choice and the stream) */
  TensorContainer(const TensorContainer<Device, dimension, DType> &other)
      : block_(NULL), rows_(0), pitch_(0), padded_(other.padded_) {
    this->PointNowhere();
    this->CloneOf(other);
  }
  ~TensorContainer(void) MSHADOW_THROW_EXCEPTION { this->Release(); }

  /*! \brief give the container this shape; the contents are undefined afterwards */
  inline void Resize(const Shape<dimension> &shape) {
    const Shape<2> flat = shape.FlatTo2D();
    if (block_ != NULL && flat[0] <= rows_ && flat[1] <= pitch_) {
      this->LookAt(shape);
    } else {
      this->TakeBlockFor(shape);
    }
  }
  inline void Resize(const Shape<dimension> &shape, DType initv) {
    this->Resize(shape);
    (*this) = initv;
  }
  /*! \brief whether blocks taken from now on have rows padded to an aligned pitch */
  inline void set_pad(bool pad) { padded_ = pad; }
  /*! \brief give the memory back; the container is empty afterwards */
  inline void Release(void) {
    if (block_ == NULL) return;
    Rows whole(block_, Shape2(rows_, pitch_));
    block_ = NULL;
    rows_ = pitch_ = 0;
    this->PointNowhere();
    FreeSpace(&whole);
  }
  /*! \brief the shape and the elements, as mshadow::SaveBinary writes a tensor */
  template <typename TStream>
  inline void SaveBinary(TStream &fo) const {  // NOLINT(*)
    mshadow::SaveBinary(fo, static_cast<const View &>(*this));
  }
  /*! \brief take the shape of the stored tensor and read its elements; returns once the
   *  elements are in place (a device container waits for its stream) */
  template <typename TStream>
  inline void LoadBinary(TStream &fi) {  // NOLINT(*)
    Tensor<cpu, dimension, DType> stored;
    mshadow::LoadBinary(fi, &stored, false);
    this->Resize(stored.shape_);
    mshadow::Copy(static_cast<View &>(*this), stored, this->stream_);
    WaitFor(this->stream_);
    FreeSpace(&stored);
  }

  inline TensorContainer &operator=(const TensorContainer<Device, dimension, DType> &other) {
    if (this != &other) {
      padded_ = other.padded_;
      this->CloneOf(other);
    }
    return *this;
  }
  inline View &operator=(DType s) { return this->__assign(s); }
  template <typename E>
  inline View &operator=(const expr::Exp<E, DType, expr::type::kMapper> &exp) {
    return this->__assign(exp);
  }
  template <typename E>
  inline View &operator=(const expr::Exp<E, DType, expr::type::kChainer> &exp) {
    return this->__assign(exp);
  }
  template <typename E>
  inline View &operator=(const expr::Exp<E, DType, expr::type::kComplex> &exp) {
    return this->__assign(exp);
  }

 private:
  DType *block_;    //!< the owned allocation (NULL: none)
  index_t rows_;    //!< its rows
  index_t pitch_;   //!< elements between the starts of its rows
  bool padded_;

  static inline void WaitFor(Stream<Device> *stream) {
    if (stream != NULL) stream->Wait();
  }
  inline void PointNowhere(void) {
    this->dptr_ = NULL;
    this->shape_[0] = 0;
    this->stride_ = 0;
  }
  /*! \brief the view of the block under `shape` (which fits it) */
  inline void LookAt(const Shape<dimension> &shape) {
    this->dptr_ = block_;
    this->shape_ = shape;
    this->stride_ = padded_ ? pitch_ : shape[dimension - 1];
  }
  inline void TakeBlockFor(const Shape<dimension> &shape) {
    this->Release();
    Rows fresh(shape.FlatTo2D());
    AllocSpace(&fresh, padded_);
    block_ = fresh.dptr_;
    rows_ = fresh.size(0);
    pitch_ = fresh.stride_;
    this->LookAt(shape);
  }
  inline void CloneOf(const TensorContainer<Device, dimension, DType> &other) {
    this->stream_ = other.stream_;
    if (other.dptr_ == NULL) return;
    this->Resize(other.shape_);
    mshadow::Copy(static_cast<View &>(*this), static_cast<const View &>(other), this->stream_);
  }
};

}  // namespace mshadow
#endif  // MSHADOW_TENSOR_CONTAINER_H_
