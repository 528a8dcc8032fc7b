/*
 * Index-remapping expression nodes: broadcast<dimcast> / repmat / broadcast_scalar,
 * reshape, swapaxis<a1, a2>, mirror, upsampling_nearest. Each is a view: no data moves
 * until the enclosing assignment evaluates it element by element, on either device,
 * through Plan::Eval below (on the GPU inside the generic map kernel).
 *
 * Semantics restate the reference's nodes of the same names
 * (mshadow/extension/broadcast.h:20-160, reshape.h:20-84, swapaxis.h:20-106, mirror.h:18-58,
 * spatial_upsampling_nearest.h:17-67), all on the flattened 2-D view (row = product of the
 * leading dimensions, column = last dimension):
 *   broadcast<d>(v, shape)   out[..., i_d, ...] = v[i_d]
 *   reshape(src, shape)      same elements in row-major order, new shape (sizes must agree)
 *   swapaxis<a1, a2>(src)    a2 < a1; out[.., i_a2, .., i_a1, ..] = src with the two swapped
 *   mirror(src)              last dimension reversed
 *   upsampling_nearest(s, k) last two dimensions repeated k times
 */
#ifndef MSHADOW_EXT_SHAPING_H_
#define MSHADOW_EXT_SHAPING_H_

#include "../core/fastdiv.h"
#include "../tensor.h"

namespace mshadow {
namespace expr {

/* ------------------------------------------------------------------ broadcast */
/*! \brief a 1-D expression repeated along every dimension but `dimdst - dimdst_m_cast` */
template <typename SrcExp, typename DType, int dimdst, int dimdst_m_cast>
struct Broadcast1DExp
    : public MakeTensorExp<Broadcast1DExp<SrcExp, DType, dimdst, dimdst_m_cast>, SrcExp, dimdst,
                           DType> {
  const SrcExp &src_;
  Broadcast1DExp(const SrcExp &src, Shape<dimdst> shape) : src_(src) { this->shape_ = shape; }
};
/*! \brief a one-element expression repeated everywhere */
template <typename SrcExp, typename DType, int dimdst>
struct BroadcastScalarExp
    : public MakeTensorExp<BroadcastScalarExp<SrcExp, DType, dimdst>, SrcExp, dimdst, DType> {
  const SrcExp &src_;
  BroadcastScalarExp(const SrcExp &src, Shape<dimdst> shape) : src_(src) { this->shape_ = shape; }
};

template <int dimcast, typename SrcExp, typename DType, int etype, int dimdst>
inline Broadcast1DExp<SrcExp, DType, dimdst, dimdst - dimcast> broadcast(
    const Exp<SrcExp, DType, etype> &src, Shape<dimdst> shape) {
  TypeCheckPass<(dimcast < dimdst) && ExpInfo<SrcExp>::kDim == 1>::
      Error_Expression_Does_Not_Meet_Dimension_Req();
  CHECK_EQ((ShapeCheck<1, SrcExp>::Check(src.self())[0]), shape[dimcast])
      << "broadcast, shape mismatch";
  return Broadcast1DExp<SrcExp, DType, dimdst, dimdst - dimcast>(src.self(), shape);
}
template <typename SrcExp, typename DType, int etype, int dimdst>
inline BroadcastScalarExp<SrcExp, DType, dimdst> broadcast_scalar(
    const Exp<SrcExp, DType, etype> &src, Shape<dimdst> shape) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim == 1>::Error_Expression_Does_Not_Meet_Dimension_Req();
  CHECK_EQ((ShapeCheck<1, SrcExp>::Check(src.self())[0]), 1U)
      << "broadcast_scalar, source need to be scalar expression";
  return BroadcastScalarExp<SrcExp, DType, dimdst>(src.self(), shape);
}
/*! \brief nrow copies of a vector stacked as the rows of a matrix */
template <typename SrcExp, typename DType, int etype>
inline Broadcast1DExp<SrcExp, DType, 2, 1> repmat(const Exp<SrcExp, DType, etype> &src,
                                                 index_t nrow) {
  return broadcast<1>(src, Shape2(nrow, ShapeCheck<1, SrcExp>::Check(src.self())[0]));
}

/* the broadcast dimension is not the last one: its index is a digit of the row number */
template <typename SrcExp, typename DType, int dimdst, int dimdst_m_cast>
struct Plan<Broadcast1DExp<SrcExp, DType, dimdst, dimdst_m_cast>, DType> {
 public:
  static const int dimcast = dimdst - dimdst_m_cast;
  explicit Plan(const Broadcast1DExp<SrcExp, DType, dimdst, dimdst_m_cast> &e)
      : src_(MakePlan(e.src_)), below_(e.shape_.ProdShape(dimcast + 1, dimdst - 1)),
        length_(e.shape_[dimcast]) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t) const {
    return src_.Eval(0, length_.Mod(below_.Div(y)));
  }
  /* one value for the whole row: a pack is that value N times */
  static const bool kPackable = true;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t) const {
    const DType v = src_.Eval(0, length_.Mod(below_.Div(y)));
    Pack<DType, N> p;
#pragma unroll
    for (int k = 0; k < N; ++k) p.v[k] = v;
    return p;
  }
  inline bool PackReady(int, index_t, bool *flat) const {
    *flat = false;
    return true;
  }

 private:
  Plan<SrcExp, DType> src_;
  const FastDivU32 below_, length_;
};
/* the broadcast dimension is the last one: its index is the column */
template <typename SrcExp, typename DType, int dimdst>
struct Plan<Broadcast1DExp<SrcExp, DType, dimdst, 1>, DType> {
 public:
  explicit Plan(const Broadcast1DExp<SrcExp, DType, dimdst, 1> &e) : src_(MakePlan(e.src_)) {}
  MSHADOW_XINLINE DType Eval(index_t, index_t x) const { return src_.Eval(0, x); }
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t, index_t x) const {
    return src_.template EvalPack<N, false>(0, x);  // every row reads it again: cached loads
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    *flat = false;
    bool ignored = true;
    return src_.PackReady(n, cols, &ignored);
  }

 private:
  Plan<SrcExp, DType> src_;
};
template <typename SrcExp, typename DType, int dimdst>
struct Plan<BroadcastScalarExp<SrcExp, DType, dimdst>, DType> {
 public:
  explicit Plan(const BroadcastScalarExp<SrcExp, DType, dimdst> &e) : src_(MakePlan(e.src_)) {}
  MSHADOW_XINLINE DType Eval(index_t, index_t) const { return src_.Eval(0, 0); }
  static const bool kPackable = true;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t, index_t) const {
    const DType v = src_.Eval(0, 0);
    Pack<DType, N> p;
#pragma unroll
    for (int k = 0; k < N; ++k) p.v[k] = v;
    return p;
  }
  inline bool PackReady(int, index_t, bool *) const { return true; }

 private:
  Plan<SrcExp, DType> src_;
};

/* ------------------------------------------------------------------ reshape */
template <typename SrcExp, typename DType, int dimdst, int dimsrc>
struct ReshapeExp
    : public MakeTensorExp<ReshapeExp<SrcExp, DType, dimdst, dimsrc>, SrcExp, dimdst, DType> {
  const SrcExp &src_;
  index_t ishapex_;  //!< last dimension of the source
  ReshapeExp(const SrcExp &src, Shape<dimdst> shape) : src_(src) {
    Shape<dimsrc> ishape = ShapeCheck<dimsrc, SrcExp>::Check(src_);
    CHECK_EQ(ishape.Size(), shape.Size()) << "reshape size must match";
    ishapex_ = ishape[dimsrc - 1];
    this->shape_ = shape;
  }
};
template <typename SrcExp, typename DType, int etype, int dimdst>
inline ReshapeExp<SrcExp, DType, dimdst, ExpInfo<SrcExp>::kDim> reshape(
    const Exp<SrcExp, DType, etype> &src, Shape<dimdst> oshape) {
  return ReshapeExp<SrcExp, DType, dimdst, ExpInfo<SrcExp>::kDim>(src.self(), oshape);
}
template <typename SrcExp, typename DType, int dimdst, int dimsrc>
struct Plan<ReshapeExp<SrcExp, DType, dimdst, dimsrc>, DType> {
 public:
  explicit Plan(const ReshapeExp<SrcExp, DType, dimdst, dimsrc> &e)
      : src_(MakePlan(e.src_)), ocols_(e.shape_[dimdst - 1]), icols_(e.ishapex_) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    const index_t flat = y * ocols_ + x;  // position in row-major order, the same on both sides
    if (dimsrc == 1) return src_.Eval(0, flat);
    const index_t row = icols_.Div(flat);
    return src_.Eval(row, flat - row * icols_.div);
  }
  /* N adjacent elements stay adjacent in the source as long as N divides both row lengths */
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    const index_t flat = y * ocols_ + x;
    if (dimsrc == 1) return src_.template EvalPack<N, STREAM>(0, flat);
    const index_t row = icols_.Div(flat);
    return src_.template EvalPack<N, STREAM>(row, flat - row * icols_.div);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    *flat = false;
    bool ignored = true;
    return ocols_ % n == 0 && icols_.div % n == 0 && src_.PackReady(n, icols_.div, &ignored);
  }

 private:
  Plan<SrcExp, DType> src_;
  const index_t ocols_;
  const FastDivU32 icols_;
};

/* ------------------------------------------------------------------ swapaxis */
/*! \brief a1 is carried as dimsrc - a1 in the type, like the reference does */
template <typename SrcExp, typename DType, int dimsrc, int m_a1, int a2>
struct SwapAxisExp
    : public MakeTensorExp<SwapAxisExp<SrcExp, DType, dimsrc, m_a1, a2>, SrcExp, dimsrc, DType> {
  static const int a1 = dimsrc - m_a1;
  const SrcExp &src_;
  explicit SwapAxisExp(const SrcExp &src) : src_(src) {
    this->shape_ = ShapeCheck<dimsrc, SrcExp>::Check(src);
    const index_t t = this->shape_[a1];
    this->shape_[a1] = this->shape_[a2];
    this->shape_[a2] = t;
  }
};
template <int a1, int a2, typename SrcExp, typename DType, int etype>
inline SwapAxisExp<SrcExp, DType, ExpInfo<SrcExp>::kDim, ExpInfo<SrcExp>::kDim - a1, a2> swapaxis(
    const Exp<SrcExp, DType, etype> &src) {
  typedef ExpInfo<SrcExp> Info;
  TypeCheckPass<(Info::kDim >= a1 + 1) && (Info::kDim >= a2 + 1) && (a2 < a1)>::
      Error_Expression_Does_Not_Meet_Dimension_Req();
  return SwapAxisExp<SrcExp, DType, Info::kDim, Info::kDim - a1, a2>(src.self());
}
/* Output dimensions, outermost first: (outer.., P = out[a2], mid.., Q = out[a1], inner..)
   where the innermost group ends with the column when a1 is not the last dimension. The
   source has Q at position a2 and P at position a1. */
template <typename SrcExp, typename DType, int dimsrc, int m_a1, int a2>
struct Plan<SwapAxisExp<SrcExp, DType, dimsrc, m_a1, a2>, DType> {
 public:
  static const int a1 = dimsrc - m_a1;
  explicit Plan(const SwapAxisExp<SrcExp, DType, dimsrc, m_a1, a2> &e)
      : src_(MakePlan(e.src_)),
        inner_(m_a1 == 1 ? 1 : e.shape_.ProdShape(a1 + 1, dimsrc - 1)),
        q_(e.shape_[a1]), mid_(e.shape_.ProdShape(a2 + 1, a1)), p_(e.shape_[a2]) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    if (m_a1 == 1) {
      /* the swapped-in dimension is the column: row = (outer, P, mid), column = Q */
      index_t rest = mid_.Div(i);
      const index_t mid = i - rest * mid_.div;
      const index_t outer = p_.Div(rest);
      const index_t p = rest - outer * p_.div;
      return src_.Eval((outer * q_.div + j) * mid_.div + mid, p);
    }
    return src_.Eval(SourceRow(i), j);
  }
  /* with the last dimension left alone the swap is a permutation of rows */
  static const bool kPackable = (m_a1 != 1) && plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t i, index_t j) const {
    return src_.template EvalPack<N, STREAM>(SourceRow(i), j);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    *flat = false;
    bool ignored = true;
    return src_.PackReady(n, cols, &ignored);
  }

 private:
  /*! \brief row of the source that holds row i of the result (a1 is not the last dimension) */
  MSHADOW_XINLINE index_t SourceRow(index_t i) const {
    index_t rest = inner_.Div(i);
    const index_t inner = i - rest * inner_.div;
    index_t next = q_.Div(rest);
    const index_t q = rest - next * q_.div;
    rest = mid_.Div(next);
    const index_t mid = next - rest * mid_.div;
    const index_t outer = p_.Div(rest);
    const index_t p = rest - outer * p_.div;
    return (((outer * q_.div + q) * mid_.div + mid) * p_.div + p) * inner_.div + inner;
  }
  Plan<SrcExp, DType> src_;
  const FastDivU32 inner_, q_, mid_, p_;
};

/* ------------------------------------------------------------------ mirror */
template <typename SrcExp, typename DType, int srcdim>
struct MirroringExp
    : public MakeTensorExp<MirroringExp<SrcExp, DType, srcdim>, SrcExp, srcdim, DType> {
  const SrcExp &src_;
  explicit MirroringExp(const SrcExp &src) : src_(src) {
    this->shape_ = ShapeCheck<srcdim, SrcExp>::Check(src_);
  }
};
template <typename SrcExp, typename DType, int etype>
inline MirroringExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> mirror(
    const Exp<SrcExp, DType, etype> &src) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return MirroringExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self());
}
template <typename SrcExp, typename DType, int srcdim>
struct Plan<MirroringExp<SrcExp, DType, srcdim>, DType> {
 public:
  explicit Plan(const MirroringExp<SrcExp, DType, srcdim> &e)
      : src_(MakePlan(e.src_)), last_(e.shape_[srcdim - 1] - 1) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const { return src_.Eval(i, last_ - j); }

 private:
  Plan<SrcExp, DType> src_;
  const index_t last_;
};

/* ------------------------------------------------------------------ upsampling_nearest */
template <typename SrcExp, typename DType, int srcdim>
struct UpSamplingNearestExp
    : public MakeTensorExp<UpSamplingNearestExp<SrcExp, DType, srcdim>, SrcExp, srcdim, DType> {
  const SrcExp &src_;
  index_t scale_;
  UpSamplingNearestExp(const SrcExp &src, index_t scale) : src_(src), scale_(scale) {
    this->shape_ = ShapeCheck<srcdim, SrcExp>::Check(src_);
    this->shape_[srcdim - 2] *= scale_;
    this->shape_[srcdim - 1] *= scale_;
  }
};
template <typename SrcExp, typename DType, int etype>
inline UpSamplingNearestExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> upsampling_nearest(
    const Exp<SrcExp, DType, etype> &src, index_t scale) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return UpSamplingNearestExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), scale);
}
template <typename SrcExp, typename DType, int srcdim>
struct Plan<UpSamplingNearestExp<SrcExp, DType, srcdim>, DType> {
 public:
  explicit Plan(const UpSamplingNearestExp<SrcExp, DType, srcdim> &e)
      : src_(MakePlan(e.src_)), scale_(e.scale_), out_h_(e.shape_[srcdim - 2]),
        src_h_(e.shape_[srcdim - 2] / e.scale_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const index_t plane = out_h_.Div(i);
    return src_.Eval(plane * src_h_ + scale_.Div(i - plane * out_h_.div), scale_.Div(j));
  }

 private:
  Plan<SrcExp, DType> src_;
  const FastDivU32 scale_, out_h_;
  const index_t src_h_;
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_SHAPING_H_
