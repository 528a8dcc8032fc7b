/*
 * pool<Reducer>(src, ky, kx, sy, sx) and unpool<Reducer>(src, pooled, grad, ky, kx, sy, sx)
 * over the last two dimensions of an expression.
 *
 * Behaviour restates mshadow/extension/spatial_pool.h:20-149 and
 * spatial_unpool.h:20-132 of the reference:
 *  - pooled size is (H - ky) / sy + 1 (floor) unless given; a window is clipped at the
 *    image edge and reduced row by row, left to right, from Reducer::SetInitValue;
 *  - unpool visits, for a source pixel, the windows covering it in (py, px) ascending
 *    order and adds PartialGrad(src, pooled) * grad, so for maximum / minimum every
 *    pixel equal to the window's result receives the gradient (equality routing).
 * On the GPU, a float tensor source with a max / min / sum reducer is recognised and
 * runs the LDS-tiled kernels; any other source runs through the generic map kernel
 * with the Eval below as its body.
 */
#ifndef MSHADOW_EXT_POOLING_H_
#define MSHADOW_EXT_POOLING_H_

#include "../core/fastdiv.h"
#include "../tensor.h"

namespace mshadow {
namespace expr {

template <typename Reducer, typename SrcExp, typename DType, int srcdim>
struct PoolingExp
    : public MakeTensorExp<PoolingExp<Reducer, SrcExp, DType, srcdim>, SrcExp, srcdim, DType> {
  const SrcExp &src_;
  index_t ksize_y_, ksize_x_;
  index_t kstride_y_, kstride_x_;
  index_t src_height_, src_width_;

  PoolingExp(const SrcExp &src, index_t ksize_y, index_t ksize_x, index_t kstride_y,
             index_t kstride_x)
      : src_(src), ksize_y_(ksize_y), ksize_x_(ksize_x), kstride_y_(kstride_y),
        kstride_x_(kstride_x) {
    Init();
    this->shape_[srcdim - 2] = (src_height_ - ksize_y) / kstride_y + 1;
    this->shape_[srcdim - 1] = (src_width_ - ksize_x) / kstride_x + 1;
  }
  PoolingExp(const SrcExp &src, Shape<2> pshape, index_t ksize_y, index_t ksize_x,
             index_t kstride_y, index_t kstride_x)
      : src_(src), ksize_y_(ksize_y), ksize_x_(ksize_x), kstride_y_(kstride_y),
        kstride_x_(kstride_x) {
    Init();
    this->shape_[srcdim - 2] = pshape[0];
    this->shape_[srcdim - 1] = pshape[1];
  }

 private:
  inline void Init() {
    Shape<srcdim> sshape = ShapeCheck<srcdim, SrcExp>::Check(src_);
    CHECK(sshape[srcdim - 1] >= ksize_x_ && sshape[srcdim - 2] >= ksize_y_)
        << "PoolingExp: kernel must be smaller than image";
    src_height_ = sshape[srcdim - 2];
    src_width_ = sshape[srcdim - 1];
    this->shape_ = sshape;
  }
};

template <typename Reducer, typename SrcExp, typename DType, int etype>
inline PoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim> pool(
    const Exp<SrcExp, DType, etype> &src, index_t ksize_y, index_t ksize_x, index_t kstride_y,
    index_t kstride_x) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return PoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), ksize_y, ksize_x,
                                                                   kstride_y, kstride_x);
}
template <typename Reducer, typename SrcExp, typename DType, int etype>
inline PoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim> pool(
    const Exp<SrcExp, DType, etype> &src, Shape<2> pshape, index_t ksize_y, index_t ksize_x,
    index_t kstride_y, index_t kstride_x) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return PoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), pshape, ksize_y,
                                                                   ksize_x, kstride_y, kstride_x);
}

template <typename Reducer, typename SrcExp, typename DType, int srcdim>
struct Plan<PoolingExp<Reducer, SrcExp, DType, srcdim>, DType> {
 public:
  explicit Plan(const PoolingExp<Reducer, SrcExp, DType, srcdim> &e)
      : src_(MakePlan(e.src_)), ky_(e.ksize_y_), kx_(e.ksize_x_), sy_(e.kstride_y_),
        sx_(e.kstride_x_), h_(e.src_height_), w_(e.src_width_), ph_(e.shape_[srcdim - 2]) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const index_t plane = ph_.Div(i);
    const index_t y0 = (i - plane * ph_.div) * sy_;
    const index_t x0 = j * sx_;
    const index_t y1 = (y0 + ky_ < h_) ? y0 + ky_ : h_;
    const index_t x1 = (x0 + kx_ < w_) ? x0 + kx_ : w_;
    DType res;
    Reducer::SetInitValue(res);
    for (index_t y = y0; y < y1; ++y) {
      for (index_t x = x0; x < x1; ++x) Reducer::Reduce(res, src_.Eval(plane * h_ + y, x));
    }
    return res;
  }

 private:
  Plan<SrcExp, DType> src_;
  const index_t ky_, kx_, sy_, sx_, h_, w_;
  const FastDivU32 ph_;
};

template <typename Reducer, typename SrcExp, typename DType, int srcdim>
struct UnPoolingExp
    : public MakeTensorExp<UnPoolingExp<Reducer, SrcExp, DType, srcdim>, SrcExp, srcdim, DType> {
  const SrcExp &data_src_;
  const SrcExp &data_pooled_;
  const SrcExp &grad_pooled_;
  index_t pshape_y_, pshape_x_;
  index_t ksize_y_, ksize_x_;
  index_t kstride_y_, kstride_x_;

  UnPoolingExp(const SrcExp &data_src, const SrcExp &data_pooled, const SrcExp &grad_pooled,
               index_t ksize_y, index_t ksize_x, index_t kstride_y, index_t kstride_x)
      : data_src_(data_src), data_pooled_(data_pooled), grad_pooled_(grad_pooled),
        ksize_y_(ksize_y), ksize_x_(ksize_x), kstride_y_(kstride_y), kstride_x_(kstride_x) {
    typedef ShapeCheck<srcdim, SrcExp> Checker;
    Shape<srcdim> pshape = Checker::Check(grad_pooled);
    CHECK_EQ(pshape, Checker::Check(data_pooled)) << "UnPoolingExp: pooled shape mismatch";
    Shape<srcdim> sshape = Checker::Check(data_src);
    for (int k = 0; k < srcdim - 2; ++k) {
      CHECK_EQ(pshape[k], sshape[k]) << "UnPoolingExp: pool and src shape mismatch";
    }
    pshape_x_ = pshape[srcdim - 1];
    pshape_y_ = pshape[srcdim - 2];
    this->shape_ = sshape;
  }
};

template <typename Reducer, typename SrcExp, typename DType, int etype>
inline UnPoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim> unpool(
    const Exp<SrcExp, DType, etype> &data_src, const Exp<SrcExp, DType, etype> &data_pooled,
    const Exp<SrcExp, DType, etype> &grad_pooled, index_t ksize_y, index_t ksize_x,
    index_t kstride_y, index_t kstride_x) {
  return UnPoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim>(
      data_src.self(), data_pooled.self(), grad_pooled.self(), ksize_y, ksize_x, kstride_y,
      kstride_x);
}

template <typename Reducer, typename SrcExp, typename DType, int srcdim>
struct Plan<UnPoolingExp<Reducer, SrcExp, DType, srcdim>, DType> {
 public:
  explicit Plan(const UnPoolingExp<Reducer, SrcExp, DType, srcdim> &e)
      : src_(MakePlan(e.data_src_)), pooled_(MakePlan(e.data_pooled_)),
        grad_(MakePlan(e.grad_pooled_)), h_(e.shape_[srcdim - 2]), ph_(e.pshape_y_),
        pw_(e.pshape_x_), ky_(e.ksize_y_), kx_(e.ksize_x_), sy_(e.kstride_y_),
        sx_(e.kstride_x_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const index_t plane = h_.Div(i);
    const index_t y = i - plane * h_.div;
    const DType vsrc = src_.Eval(i, j);
    /* first and one-past-last window index whose extent [p*s, p*s + k) contains the pixel */
    const index_t py0 = y < ky_ ? 0 : sy_.Div(y - ky_ + sy_.div);
    const index_t px0 = j < kx_ ? 0 : sx_.Div(j - kx_ + sx_.div);
    index_t py1 = sy_.Div(y + sy_.div);
    index_t px1 = sx_.Div(j + sx_.div);
    if (py1 > ph_) py1 = ph_;
    if (px1 > pw_) px1 = pw_;
    DType val = static_cast<DType>(0);
    for (index_t py = py0; py < py1; ++py) {
      for (index_t px = px0; px < px1; ++px) {
        val += Reducer::PartialGrad(vsrc, pooled_.Eval(plane * ph_ + py, px)) *
               grad_.Eval(plane * ph_ + py, px);
      }
    }
    return val;
  }

 private:
  Plan<SrcExp, DType> src_, pooled_, grad_;
  const FastDivU32 h_;
  const index_t ph_, pw_, ky_, kx_;
  const FastDivU32 sy_, sx_;
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_POOLING_H_
