/*
 * Convolution data movement as expressions:
 *   unpack_patch2col(img, ky, kx, stride, dilate)          image -> column matrix
 *   pack_col2patch(col, imshape, ky, kx, stride, dilate)   column matrix -> image (sums overlaps)
 *   pad(src, pad_y, pad_x)                                 zero border on the last two dims
 *   crop(src, oshape [, start_y, start_x])                 window of the last two dims
 *
 * Index conventions restate mshadow/extension/unpack_patch2col.h:20-148,
 * pack_col2patch.h:21-151, pad.h:18-108 and crop.h:18-116 of the reference:
 *   col row  = (c * ky + dy) * kx + dx            col column = (n * OH + oy) * OW + ox
 *   OH = (H - (dil_y * (ky - 1) + 1)) / stride_y + 1 (likewise OW)
 * pack_col2patch adds the covering patches in (py, px) ascending order in the element
 * type, so half_t sums round after every addition. "Convolution padding" is spelled
 * unpack_patch2col(pad(img, p), ...) and crop(pack_col2patch(...), shape, p, p); on the
 * GPU those two compositions over plain tensors are recognised and run as single
 * kernels.
 */
#ifndef MSHADOW_EXT_PATCHES_H_
#define MSHADOW_EXT_PATCHES_H_

#include "../core/fastdiv.h"
#include "../tensor.h"

namespace mshadow {
namespace expr {

/* ------------------------------------------------------------------ pad */
template <typename SrcExp, typename DType, int srcdim>
struct PaddingExp : public MakeTensorExp<PaddingExp<SrcExp, DType, srcdim>, SrcExp, srcdim, DType> {
  const SrcExp &src_;
  index_t pad_y_, pad_x_;
  index_t src_height_, src_width_;
  PaddingExp(const SrcExp &src, index_t pad_y, index_t pad_x)
      : src_(src), pad_y_(pad_y), pad_x_(pad_x) {
    this->shape_ = ShapeCheck<srcdim, SrcExp>::Check(src_);
    src_height_ = this->shape_[srcdim - 2];
    src_width_ = this->shape_[srcdim - 1];
    this->shape_[srcdim - 2] += pad_y * 2;
    this->shape_[srcdim - 1] += pad_x * 2;
  }
};
template <typename SrcExp, typename DType, int etype>
inline PaddingExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> pad(const Exp<SrcExp, DType, etype> &src,
                                                            index_t pad) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return PaddingExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), pad, pad);
}
template <typename SrcExp, typename DType, int etype>
inline PaddingExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> pad(const Exp<SrcExp, DType, etype> &src,
                                                            index_t pad_y, index_t pad_x) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return PaddingExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), pad_y, pad_x);
}
template <typename SrcExp, typename DType, int srcdim>
struct Plan<PaddingExp<SrcExp, DType, srcdim>, DType> {
 public:
  explicit Plan(const PaddingExp<SrcExp, DType, srcdim> &e)
      : src_(MakePlan(e.src_)), pad_y_(e.pad_y_), pad_x_(e.pad_x_),
        new_height_(e.shape_[srcdim - 2]), src_height_(e.src_height_),
        src_width_(e.src_width_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const index_t plane = new_height_.Div(i);
    const index_t y = i - plane * new_height_.div;
    if (y < pad_y_ || j < pad_x_) return static_cast<DType>(0);
    const index_t h = y - pad_y_;
    const index_t w = j - pad_x_;
    if (h >= src_height_ || w >= src_width_) return static_cast<DType>(0);
    return src_.Eval(plane * src_height_ + h, w);
  }

 private:
  Plan<SrcExp, DType> src_;
  const index_t pad_y_, pad_x_;
  const FastDivU32 new_height_;
  const index_t src_height_, src_width_;
};

/* ------------------------------------------------------------------ crop */
template <typename SrcExp, typename DType, int srcdim>
struct CroppingExp : public MakeTensorExp<CroppingExp<SrcExp, DType, srcdim>, SrcExp, srcdim, DType> {
  const SrcExp &src_;
  index_t pad_height_, pad_width_;
  index_t src_height_;
  /*! \brief centred crop */
  explicit CroppingExp(const SrcExp &src, Shape<2> cshape) : src_(src) {
    this->shape_ = ShapeCheck<srcdim, SrcExp>::Check(src_);
    CHECK_GE(this->shape_[srcdim - 2], cshape[0]) << "CroppingExp: height requirement not met";
    CHECK_GE(this->shape_[srcdim - 1], cshape[1]) << "CroppingExp: width requirement not met";
    pad_height_ = (this->shape_[srcdim - 2] - cshape[0]) / 2;
    pad_width_ = (this->shape_[srcdim - 1] - cshape[1]) / 2;
    Finish(cshape);
  }
  /*! \brief crop starting at (start_height, start_width) */
  explicit CroppingExp(const SrcExp &src, Shape<2> cshape, index_t start_height,
                       index_t start_width)
      : src_(src), pad_height_(start_height), pad_width_(start_width) {
    this->shape_ = ShapeCheck<srcdim, SrcExp>::Check(src_);
    CHECK_GE(this->shape_[srcdim - 2], cshape[0] + start_height)
        << "CroppingExp: height requirement not met";
    CHECK_GE(this->shape_[srcdim - 1], cshape[1] + start_width)
        << "CroppingExp: width requirement not met";
    Finish(cshape);
  }

 private:
  inline void Finish(Shape<2> cshape) {
    src_height_ = this->shape_[srcdim - 2];
    this->shape_[srcdim - 2] = cshape[0];
    this->shape_[srcdim - 1] = cshape[1];
  }
};
template <typename SrcExp, typename DType, int etype>
inline CroppingExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> crop(const Exp<SrcExp, DType, etype> &src,
                                                              Shape<2> oshape) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return CroppingExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), oshape);
}
template <typename SrcExp, typename DType, int etype>
inline CroppingExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> crop(const Exp<SrcExp, DType, etype> &src,
                                                              Shape<2> oshape,
                                                              index_t start_height,
                                                              index_t start_width) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return CroppingExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), oshape, start_height,
                                                           start_width);
}
template <typename SrcExp, typename DType, int srcdim>
struct Plan<CroppingExp<SrcExp, DType, srcdim>, DType> {
 public:
  explicit Plan(const CroppingExp<SrcExp, DType, srcdim> &e)
      : src_(MakePlan(e.src_)), off_y_(e.pad_height_), off_x_(e.pad_width_),
        new_height_(e.shape_[srcdim - 2]), src_height_(e.src_height_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const index_t plane = new_height_.Div(i);
    const index_t y = i - plane * new_height_.div;
    return src_.Eval(plane * src_height_ + y + off_y_, j + off_x_);
  }

 private:
  Plan<SrcExp, DType> src_;
  const index_t off_y_, off_x_;
  const FastDivU32 new_height_;
  const index_t src_height_;
};

/* ------------------------------------------------------------------ unpack_patch2col */
template <typename SrcExp, typename DType, int srcdim>
struct UnpackPatchToColXExp
    : public MakeTensorExp<UnpackPatchToColXExp<SrcExp, DType, srcdim>, SrcExp, 2, DType> {
  const SrcExp &img_;
  index_t psize_y_, psize_x_;
  index_t pstride_y_, pstride_x_;
  index_t pdilate_y_, pdilate_x_;
  index_t i_channel_, i_height_, i_width_;
  UnpackPatchToColXExp(const SrcExp &img, index_t psize_y, index_t psize_x, index_t pstride_y,
                       index_t pstride_x, index_t pdilate_y, index_t pdilate_x)
      : img_(img), psize_y_(psize_y), psize_x_(psize_x), pstride_y_(pstride_y),
        pstride_x_(pstride_x), pdilate_y_(pdilate_y), pdilate_x_(pdilate_x) {
    Shape<srcdim> imshape = ShapeCheck<srcdim, SrcExp>::Check(img_);
    CHECK(imshape[srcdim - 1] >= psize_x && imshape[srcdim - 2] >= psize_y)
        << "UnpackPatchToCol:image shape smaller than patch size";
    i_channel_ = imshape[srcdim - 3];
    i_height_ = imshape[srcdim - 2];
    i_width_ = imshape[srcdim - 1];
    const index_t num = imshape.ProdShape(0, srcdim - 3);
    const index_t o_height = (i_height_ - (pdilate_y * (psize_y - 1) + 1)) / pstride_y + 1;
    const index_t o_width = (i_width_ - (pdilate_x * (psize_x - 1) + 1)) / pstride_x + 1;
    this->shape_[1] = o_height * o_width * num;
    this->shape_[0] = psize_y * psize_x * i_channel_;
  }
};
template <typename SrcExp, typename DType, int etype>
inline UnpackPatchToColXExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> unpack_patch2col(
    const Exp<SrcExp, DType, etype> &img, index_t psize_y, index_t psize_x, index_t pstride,
    index_t pdilate) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 3>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return UnpackPatchToColXExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(
      img.self(), psize_y, psize_x, pstride, pstride, pdilate, pdilate);
}
template <typename SrcExp, typename DType, int etype>
inline UnpackPatchToColXExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> unpack_patch2col(
    const Exp<SrcExp, DType, etype> &img, index_t psize_y, index_t psize_x, index_t pstride_y_,
    index_t pstride_x_, index_t pdilate_y_, index_t pdilate_x_) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 3>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return UnpackPatchToColXExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(
      img.self(), psize_y, psize_x, pstride_y_, pstride_x_, pdilate_y_, pdilate_x_);
}
template <typename SrcExp, typename DType, int srcdim>
struct Plan<UnpackPatchToColXExp<SrcExp, DType, srcdim>, DType> {
 public:
  explicit Plan(const UnpackPatchToColXExp<SrcExp, DType, srcdim> &e)
      : src_(MakePlan(e.img_)), ky_(e.psize_y_), kx_(e.psize_x_), sy_(e.pstride_y_),
        sx_(e.pstride_x_), dy_(e.pdilate_y_), dx_(e.pdilate_x_), ch_(e.i_channel_),
        h_(e.i_height_), w_(e.i_width_),
        oh_((h_ - (dy_ * (e.psize_y_ - 1) + 1)) / sy_ + 1),
        ow_((w_ - (dx_ * (e.psize_x_ - 1) + 1)) / sx_ + 1) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    /* row i -> (channel, tap y, tap x); column j -> (image, out y, out x) */
    const index_t i_rest = kx_.Div(i);
    const index_t tap_x = (i - i_rest * kx_.div) * dx_;
    const index_t c = ky_.Div(i_rest);
    const index_t tap_y = (i_rest - c * ky_.div) * dy_;
    const index_t j_rest = ow_.Div(j);
    const index_t x = (j - j_rest * ow_.div) * sx_ + tap_x;
    const index_t n = oh_.Div(j_rest);
    const index_t y = (j_rest - n * oh_.div) * sy_ + tap_y;
    if (x < w_ && y < h_) return src_.Eval((n * ch_ + c) * h_ + y, x);
    return DType(0.0f);
  }

 private:
  Plan<SrcExp, DType> src_;
  /* members in order of initialisation; the divisors of Eval as multiply-high constants */
  const FastDivU32 ky_, kx_;
  const index_t sy_, sx_, dy_, dx_, ch_, h_, w_;
  const FastDivU32 oh_, ow_;
};

/* ------------------------------------------------------------------ pack_col2patch */
template <typename SrcExp, typename DType, int dstdim>
struct PackColToPatchXExp
    : public MakeTensorExp<PackColToPatchXExp<SrcExp, DType, dstdim>, SrcExp, dstdim, DType> {
  const SrcExp &src_;
  index_t psize_y_, psize_x_;
  index_t pstride_y_, pstride_x_;
  index_t pdilate_y_, pdilate_x_;
  PackColToPatchXExp(const SrcExp &src, Shape<dstdim> imshape, index_t psize_y, index_t psize_x,
                     index_t pstride_y, index_t pstride_x, index_t pdilate_y, index_t pdilate_x)
      : src_(src), psize_y_(psize_y), psize_x_(psize_x), pstride_y_(pstride_y),
        pstride_x_(pstride_x), pdilate_y_(pdilate_y), pdilate_x_(pdilate_x) {
    this->shape_ = imshape;
    const index_t o_height =
        (imshape[dstdim - 2] - (pdilate_y * (psize_y - 1) + 1)) / pstride_y + 1;
    const index_t o_width =
        (imshape[dstdim - 1] - (pdilate_x * (psize_x - 1) + 1)) / pstride_x + 1;
    Shape<2> sshape = ShapeCheck<2, SrcExp>::Check(src_);
    CHECK_EQ(sshape[1], o_height * o_width * imshape.ProdShape(0, dstdim - 3))
        << "PackColToPatchExp: src.size(1) mismatch";
    CHECK_EQ(sshape[0], psize_y * psize_x * imshape[dstdim - 3])
        << "PackColToPatchExp: src.size(0) mismatch";
  }
};
template <typename SrcExp, typename DType, int dstdim, int etype>
inline PackColToPatchXExp<SrcExp, DType, dstdim> pack_col2patch(
    const expr::Exp<SrcExp, DType, etype> &src, Shape<dstdim> imshape, index_t psize_y,
    index_t psize_x, index_t pstride, index_t pdilate) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim == 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  CHECK(imshape[dstdim - 1] >= psize_x && imshape[dstdim - 2] >= psize_y)
      << "PackColToPatch:image shape smaller than patch size";
  return PackColToPatchXExp<SrcExp, DType, dstdim>(src.self(), imshape, psize_y, psize_x, pstride,
                                                   pstride, pdilate, pdilate);
}
template <typename SrcExp, typename DType, int dstdim, int etype>
inline PackColToPatchXExp<SrcExp, DType, dstdim> pack_col2patch(
    const expr::Exp<SrcExp, DType, etype> &src, Shape<dstdim> imshape, index_t psize_y,
    index_t psize_x, index_t pstride_y, index_t pstride_x, index_t pdilate_y,
    index_t pdilate_x) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim == 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  CHECK(imshape[dstdim - 1] >= psize_x && imshape[dstdim - 2] >= psize_y)
      << "PackColToPatch:image shape smaller than patch size";
  return PackColToPatchXExp<SrcExp, DType, dstdim>(src.self(), imshape, psize_y, psize_x,
                                                   pstride_y, pstride_x, pdilate_y, pdilate_x);
}
template <typename SrcExp, typename DType, int dstdim>
struct Plan<PackColToPatchXExp<SrcExp, DType, dstdim>, DType> {
 public:
  explicit Plan(const PackColToPatchXExp<SrcExp, DType, dstdim> &e)
      : src_(MakePlan(e.src_)), ky_(e.psize_y_), kx_(e.psize_x_), sy_(e.pstride_y_),
        sx_(e.pstride_x_), dy_(e.pdilate_y_), dx_(e.pdilate_x_), ch_(e.shape_[dstdim - 3]),
        h_(e.shape_[dstdim - 2]),
        oh_((e.shape_[dstdim - 2] - (dy_.div * (ky_ - 1) + 1)) / sy_.div + 1),
        ow_((e.shape_[dstdim - 1] - (dx_.div * (kx_ - 1) + 1)) / sx_.div + 1) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const index_t i_rest = h_.Div(i);
    const index_t y = i - i_rest * h_.div;
    const index_t n = ch_.Div(i_rest);
    const index_t c = i_rest - n * ch_.div;
    const index_t x = j;
    const index_t sy = sy_.div, sx = sx_.div, dy = dy_.div, dx = dx_.div;
    const index_t span_y = dy * (ky_ - 1) + 1;
    const index_t span_x = dx * (kx_ - 1) + 1;
    /* patches whose (dilated) extent reaches this pixel */
    const index_t py0 = y < span_y ? dy_.Mod(y) : sy_.Div(y - span_y + sy);
    const index_t px0 = x < span_x ? dx_.Mod(x) : sx_.Div(x - span_x + sx);
    index_t py1 = sy_.Div(y + sy);
    index_t px1 = sx_.Div(x + sx);
    if (py1 > oh_) py1 = oh_;
    if (px1 > ow_) px1 = ow_;
    DType res = static_cast<DType>(0);
    for (index_t py = py0; py < py1; py += dy) {
      for (index_t px = px0; px < px1; px += dx) {
        res += src_.Eval((c * ky_ + dy_.Div(y - py * sy)) * kx_ + dx_.Div(x - px * sx),
                         (n * oh_ + py) * ow_ + px);
      }
    }
    return res;
  }

 private:
  Plan<SrcExp, DType> src_;
  const index_t ky_, kx_;
  const FastDivU32 sy_, sx_, dy_, dx_, ch_, h_;
  const index_t oh_, ow_;
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_PATCHES_H_
