/*
 * Expression nodes that address one axis (or a permutation of the axes) of a tensor:
 *   reduce_with_axis<Reducer, mask>(src, axis) / reduce_keepdim   reduce one axis away
 *   broadcast_with_axis(src, axis, size) / broadcast_keepdim      insert / widen one axis
 *   broadcast_multi_axes(src, axes, sizes) / broadcast_to          widen several size-1 axes
 *   transpose(src, axes) / transpose_indices(idx, shape, axes)     permute the axes
 *   concat<dim>(a, b), slice<dim>(src, begin, end),
 *   slice(src, begin, end) with one range per axis, flip(src, dim)  views that can also be
 *                                                                   assigned to
 *
 * Semantics restate the reference's nodes of the same names (mshadow/extension/
 * reduce_with_axis.h:14-131, broadcast_with_axis.h:17-258, transpose.h:14-200,
 * concat.h:14-194, slice.h:14-156, slice_ex.h:14-135, flip.h:14-132). All index
 * arithmetic is on the flattened 2-D view (row = product of the leading dimensions,
 * column = last dimension); divisors are constants of the node, so the plans divide by
 * multiply-high.
 *
 * reduce_with_axis walks the axis in ascending order from Reducer::SetInitValue; with
 * mask = true it returns, as DType, the last position at which the running result
 * changed (arg-max / arg-min of the first extremum, 0 if nothing ever changed).
 */
#ifndef MSHADOW_EXT_AXES_H_
#define MSHADOW_EXT_AXES_H_

#include <vector>

#include "../core/fastdiv.h"
#include "../tensor.h"

namespace mshadow {
namespace expr {

namespace axes_detail {
/*! \brief evaluates a plan at a flat row-major position of its expression */
struct FlatAt {
  FastDivU32 last;  //!< length of the expression's last dimension
  FlatAt() {}
  explicit FlatAt(index_t last_dim) : last(last_dim) {}
  template <typename P>
  MSHADOW_XINLINE auto Eval(const P &plan, index_t flat) const -> decltype(plan.Eval(0, 0)) {
    const index_t row = last.Div(flat);
    return plan.Eval(row, flat - row * last.div);
  }
  template <typename P>
  MSHADOW_XINLINE auto REval(P &plan, index_t flat) const -> decltype(plan.REval(0, 0)) {
    const index_t row = last.Div(flat);
    return plan.REval(row, flat - row * last.div);
  }
};
/*! \brief a row number taken apart into the digits of dimensions 0 .. dim-2 */
template <int dim>
struct RowDigits {
  FastDivU32 len[dim > 1 ? dim - 1 : 1];
  RowDigits() {}
  explicit RowDigits(const Shape<dim> &shape) {
    for (int k = 0; k + 1 < dim; ++k) len[k] = FastDivU32(shape[k]);
  }
  /*! \brief digit of dimension k, removing it from `rest` (call with k descending) */
  MSHADOW_XINLINE index_t Pop(int k, index_t &rest) const {
    const index_t q = len[k].Div(rest);
    const index_t digit = rest - q * len[k].div;
    rest = q;
    return digit;
  }
};
/*! \brief PackReady of a source plan for a node that needs real row numbers itself */
template <typename P>
inline bool SourcePackReady(const P &plan, int n, index_t cols, bool *flat) {
  *flat = false;
  bool ignored = true;
  return plan.PackReady(n, cols, &ignored);
}
}  // namespace axes_detail

/* ------------------------------------------------------------------ reduce_with_axis */
template <typename Reducer, typename SrcExp, typename DType, int dimsrc, bool mask, int dimdst>
struct ReduceWithAxisExp
    : public MakeTensorExp<ReduceWithAxisExp<Reducer, SrcExp, DType, dimsrc, mask, dimdst>, SrcExp,
                           dimdst, DType> {
  const SrcExp &src_;
  index_t last_dst_dim_;  //!< last dimension of the result
  index_t trailing_;      //!< elements spanned by the dimensions after the axis
  index_t size_;          //!< length of the axis
  index_t last_;          //!< last dimension of the source
  ReduceWithAxisExp(const SrcExp &src, int axis) : src_(src) {
    const bool keepdim = (dimsrc == dimdst);
    CHECK(dimsrc > axis) << "reduce axis out of bound";
    Shape<dimsrc> sshape = ShapeCheck<dimsrc, SrcExp>::Check(src_);
    for (int i = 0; i < axis; ++i) this->shape_[i] = sshape[i];
    size_ = sshape[axis];
    trailing_ = 1;
    if (keepdim) this->shape_[axis] = 1;
    for (int i = axis + 1; i < dimsrc; ++i) {
      trailing_ *= sshape[i];
      this->shape_[keepdim ? i : i - 1] = sshape[i];
    }
    last_ = sshape[dimsrc - 1];
    last_dst_dim_ = this->shape_[dimdst - 1];
  }
};
template <typename Reducer, bool mask, typename SrcExp, typename DType, int etype>
inline ReduceWithAxisExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim, mask,
                         ExpInfo<SrcExp>::kDim - 1>
reduce_with_axis(const Exp<SrcExp, DType, etype> &src, int axis) {
  return ReduceWithAxisExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim, mask,
                           ExpInfo<SrcExp>::kDim - 1>(src.self(), axis);
}
template <typename Reducer, bool mask, typename SrcExp, typename DType, int etype>
inline ReduceWithAxisExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim, mask,
                         ExpInfo<SrcExp>::kDim>
reduce_keepdim(const Exp<SrcExp, DType, etype> &src, int axis) {
  return ReduceWithAxisExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim, mask,
                           ExpInfo<SrcExp>::kDim>(src.self(), axis);
}
template <typename Reducer, typename SrcExp, typename DType, int dimsrc, bool mask, int dimdst>
struct Plan<ReduceWithAxisExp<Reducer, SrcExp, DType, dimsrc, mask, dimdst>, DType> {
 public:
  explicit Plan(const ReduceWithAxisExp<Reducer, SrcExp, DType, dimsrc, mask, dimdst> &e)
      : src_(MakePlan(e.src_)), at_(e.last_), last_dst_dim_(e.last_dst_dim_),
        trailing_(e.trailing_), size_(e.size_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const index_t flat = i * last_dst_dim_ + j;
    const index_t outer = trailing_.Div(flat);
    const index_t inner = flat - outer * trailing_.div;
    index_t z = outer * size_ * trailing_.div + inner;  // first element along the axis
    DType res;
    Reducer::SetInitValue(res);
    index_t where = 0;
    for (index_t k = 0; k < size_; ++k, z += trailing_.div) {
      const DType before = res;
      Reducer::Reduce(res, at_.Eval(src_, z));
      if (mask && before != res) where = k;
    }
    return mask ? static_cast<DType>(static_cast<int>(where)) : res;
  }
  /* when the reduced axis is not the last one, the elements along it sit in different rows of
     the source at the same column: N adjacent columns are reduced side by side */
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t i, index_t j) const {
    const index_t flat = i * last_dst_dim_ + j;
    const index_t outer = trailing_.Div(flat);
    const index_t inner = flat - outer * trailing_.div;
    index_t row = at_.last.Div(outer * size_ * trailing_.div + inner);
    const index_t row_step = at_.last.Div(trailing_.div);
    Pack<DType, N> res;
    index_t where[N];
#pragma unroll
    for (int c = 0; c < N; ++c) {
      Reducer::SetInitValue(res.v[c]);
      where[c] = 0;
    }
    for (index_t k = 0; k < size_; ++k, row += row_step) {
      const Pack<DType, N> v = src_.template EvalPack<N, STREAM>(row, j);
#pragma unroll
      for (int c = 0; c < N; ++c) {
        const DType before = res.v[c];
        Reducer::Reduce(res.v[c], v.v[c]);
        if (mask && before != res.v[c]) where[c] = k;
      }
    }
    if (mask) {
#pragma unroll
      for (int c = 0; c < N; ++c) res.v[c] = static_cast<DType>(static_cast<int>(where[c]));
    }
    return res;
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    const index_t last = at_.last.div;
    return axes_detail::SourcePackReady(src_, n, cols, flat) && last_dst_dim_ == last &&
           trailing_.div % last == 0;
  }

 private:
  Plan<SrcExp, DType> src_;
  const axes_detail::FlatAt at_;
  const index_t last_dst_dim_;
  const FastDivU32 trailing_;
  const index_t size_;
};

/* ------------------------------------------------------------------ broadcast_with_axis */
template <typename SrcExp, typename DType, int dimsrc, int dimdst>
struct BroadcastWithAxisExp
    : public MakeTensorExp<BroadcastWithAxisExp<SrcExp, DType, dimsrc, dimdst>, SrcExp, dimdst,
                           DType> {
  const SrcExp &src_;
  index_t dst_last_, trailing_, size_, last_;
  BroadcastWithAxisExp(const SrcExp &src, const int axis, const index_t size)
      : src_(src), size_(size) {
    const bool keepdim = (dimsrc == dimdst);
    Shape<dimsrc> sshape = ShapeCheck<dimsrc, SrcExp>::Check(src_);
    trailing_ = 1;
    if (!keepdim) {
      /* the new axis goes after `axis` (-1: in front) */
      CHECK(dimsrc > axis && axis >= -1)
          << "broadcast axis (no keepdim) out of bound, axis must be between -1 and"
          << dimsrc - 1 << ", given=" << axis << ".";
      for (int i = 0; i <= axis; ++i) this->shape_[i] = sshape[i];
      this->shape_[axis + 1] = size_;
      for (int i = axis + 1; i < dimsrc; ++i) {
        trailing_ *= sshape[i];
        this->shape_[i + 1] = sshape[i];
      }
    } else {
      CHECK(dimdst > axis && axis >= 0)
          << "broadcast axis (keepdim) out of bound, axis must be between 0 and" << dimdst - 1
          << ", given=" << axis << ".";
      CHECK_EQ(sshape[axis], 1U)
          << "Size of the dimension of the broadcasting axis must be 1 when keepdim is on, "
          << "src_shape[" << axis << "]=" << sshape[axis] << ".";
      for (int i = 0; i < axis; ++i) this->shape_[i] = sshape[i];
      this->shape_[axis] = size_;
      for (int i = axis + 1; i < dimdst; ++i) {
        trailing_ *= sshape[i];
        this->shape_[i] = sshape[i];
      }
    }
    last_ = sshape[dimsrc - 1];
    dst_last_ = this->shape_[dimdst - 1];
  }
};
template <typename SrcExp, typename DType, int etype>
inline BroadcastWithAxisExp<SrcExp, DType, ExpInfo<SrcExp>::kDim, ExpInfo<SrcExp>::kDim + 1>
broadcast_with_axis(const Exp<SrcExp, DType, etype> &src, const int axis, const index_t size) {
  return BroadcastWithAxisExp<SrcExp, DType, ExpInfo<SrcExp>::kDim, ExpInfo<SrcExp>::kDim + 1>(
      src.self(), axis, size);
}
template <typename SrcExp, typename DType, int etype>
inline BroadcastWithAxisExp<SrcExp, DType, ExpInfo<SrcExp>::kDim, ExpInfo<SrcExp>::kDim>
broadcast_keepdim(const Exp<SrcExp, DType, etype> &src, const int axis, const index_t size) {
  return BroadcastWithAxisExp<SrcExp, DType, ExpInfo<SrcExp>::kDim, ExpInfo<SrcExp>::kDim>(
      src.self(), axis, size);
}
template <typename SrcExp, typename DType, int dimsrc, int dimdst>
struct Plan<BroadcastWithAxisExp<SrcExp, DType, dimsrc, dimdst>, DType> {
 public:
  explicit Plan(const BroadcastWithAxisExp<SrcExp, DType, dimsrc, dimdst> &e)
      : src_(MakePlan(e.src_)), at_(e.last_), dst_last_(e.dst_last_), trailing_(e.trailing_),
        size_(e.size_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const index_t flat = i * dst_last_ + j;
    const index_t upper = trailing_.Div(flat);  // (outer, position on the new axis)
    const index_t inner = flat - upper * trailing_.div;
    return at_.Eval(src_, size_.Div(upper) * trailing_.div + inner);
  }
  /* a new axis in front of the last dimension repeats whole rows */
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t i, index_t j) const {
    const index_t flat = i * dst_last_ + j;
    const index_t upper = trailing_.Div(flat);
    const index_t inner = flat - upper * trailing_.div;
    return src_.template EvalPack<N, false>(at_.last.Div(size_.Div(upper) * trailing_.div + inner),
                                            j);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    const index_t last = at_.last.div;
    return axes_detail::SourcePackReady(src_, n, cols, flat) && dst_last_ == last &&
           trailing_.div % last == 0;
  }

 private:
  Plan<SrcExp, DType> src_;
  const axes_detail::FlatAt at_;
  const index_t dst_last_;
  const FastDivU32 trailing_, size_;
};

/*! \brief several size-1 axes widened at once; axes ascending, sizes[i] for axes[i] */
template <typename SrcExp, typename DType, int dimsrc>
struct BroadcastWithMultiAxesExp
    : public MakeTensorExp<BroadcastWithMultiAxesExp<SrcExp, DType, dimsrc>, SrcExp, dimsrc,
                           DType> {
  const SrcExp &src_;
  index_t dst_last_, axesnum_, last_;
  Shape<dimsrc> trailings_, sizes_;
  template <typename TShape>
  BroadcastWithMultiAxesExp(const SrcExp &src, const TShape &axes, const TShape &sizes)
      : src_(src) {
    Shape<dimsrc> sshape = ShapeCheck<dimsrc, SrcExp>::Check(src_);
    CHECK(axes.ndim() == sizes.ndim()) << "ndim of axes and sizes must be equal.";
    axesnum_ = axes.ndim();
    CHECK(axesnum_ <= dimsrc) << "Number of broadcasting axes must be smaller than"
                                 "the source ndim, number of axes=" << axesnum_
                              << " dimsrc=" << dimsrc;
    for (index_t i = 0; i < axesnum_; i++) {
      CHECK(dimsrc > axes[i]) << "broadcast axis (keepdim) out of bound, all axes must be between"
                                 " 0 and" << dimsrc - 1 << ", given axes[" << i
                              << "] = " << axes[i] << ".";
      CHECK_EQ(sshape[axes[i]], 1U) << "Size of the dimension of the broadcasting axis must be 1"
                                    << ", src_shape[" << axes[i] << "]=" << sshape[axes[i]] << ".";
      if (i + 1 < axesnum_) {
        CHECK(axes[i] < axes[i + 1]) << "The given axes must be in increasing order.";
      }
    }
    for (index_t i = 0; i < dimsrc; i++) {
      this->shape_[i] = sshape[i];
      sizes_[i] = 1;
      trailings_[i] = 1;
    }
    for (index_t i = 0; i < axesnum_; i++) {
      this->shape_[axes[i]] = sizes[i];
      sizes_[i] = sizes[i];
    }
    for (index_t i = 0; i < axesnum_; i++) {
      for (index_t j = axes[i] + 1; j < dimsrc; ++j) trailings_[i] *= this->shape_[j];
    }
    last_ = sshape[dimsrc - 1];
    dst_last_ = this->shape_[dimsrc - 1];
  }
};
template <typename SrcExp, typename DType, int etype, typename TShape>
inline BroadcastWithMultiAxesExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> broadcast_multi_axes(
    const Exp<SrcExp, DType, etype> &src, const TShape &axes, const TShape &sizes) {
  return BroadcastWithMultiAxesExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), axes, sizes);
}
/*! \brief widen every size-1 axis whose target length differs */
template <typename SrcExp, typename DType, int etype, typename TShape>
inline BroadcastWithMultiAxesExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> broadcast_to(
    const Exp<SrcExp, DType, etype> &src, const TShape &target_shape) {
  static const size_t dimsrc = ExpInfo<SrcExp>::kDim;
  CHECK_EQ(target_shape.ndim(), dimsrc);
  std::vector<index_t> axes_vec, sizes_vec;
  Shape<dimsrc> sshape = ShapeCheck<dimsrc, SrcExp>::Check(src.self());
  for (size_t i = 0; i < dimsrc; ++i) {
    if (sshape[i] != target_shape[i]) {
      CHECK_EQ(sshape[i], 1U) << "broadcasting axis must have size 1, received shape=" << sshape
                              << " target_shape=" << target_shape;
      axes_vec.push_back(i);
      sizes_vec.push_back(target_shape[i]);
    }
  }
  TShape axes = TShape(axes_vec.begin(), axes_vec.end());
  TShape sizes = TShape(sizes_vec.begin(), sizes_vec.end());
  return BroadcastWithMultiAxesExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), axes, sizes);
}
template <typename SrcExp, typename DType, int dimsrc>
struct Plan<BroadcastWithMultiAxesExp<SrcExp, DType, dimsrc>, DType> {
 public:
  explicit Plan(const BroadcastWithMultiAxesExp<SrcExp, DType, dimsrc> &e)
      : src_(MakePlan(e.src_)), at_(e.last_), dst_last_(e.dst_last_), axesnum_(e.axesnum_) {
    for (int p = 0; p < dimsrc; ++p) {
      trailings_[p] = FastDivU32(e.trailings_[p]);
      sizes_[p] = FastDivU32(e.sizes_[p]);
    }
  }
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    index_t flat = i * dst_last_ + j;
    /* squeeze the widened axes out again, outermost first */
    for (index_t p = 0; p < static_cast<index_t>(dimsrc) && p < axesnum_; ++p) {
      const index_t upper = trailings_[p].Div(flat);
      flat = sizes_[p].Div(upper) * trailings_[p].div + (flat - upper * trailings_[p].div);
    }
    return at_.Eval(src_, flat);
  }

 private:
  Plan<SrcExp, DType> src_;
  const axes_detail::FlatAt at_;
  const index_t dst_last_, axesnum_;
  FastDivU32 trailings_[dimsrc], sizes_[dimsrc];
};

/* ------------------------------------------------------------------ transpose */
/*! \brief result dimension i is source dimension axes[i] */
template <typename SrcExp, typename DType, int dimsrc>
struct TransposeExExp
    : public MakeTensorExp<TransposeExExp<SrcExp, DType, dimsrc>, SrcExp, dimsrc, DType> {
  const SrcExp &src_;
  const Shape<dimsrc> axes_;
  Shape<dimsrc> dst_in_src_stride_;  //!< distance in the source of a step along each result axis
  index_t src_stride_;               //!< last dimension of the source
  TransposeExExp(const SrcExp &src, Shape<dimsrc> axes) : src_(src), axes_(axes) {
    Shape<dimsrc> sshape = ShapeCheck<dimsrc, SrcExp>::Check(src);
    src_stride_ = sshape[dimsrc - 1];
    Shape<dimsrc> step;
    step[dimsrc - 1] = 1;
    for (int i = dimsrc - 2; i >= 0; --i) step[i] = sshape[i + 1] * step[i + 1];
    for (int i = 0; i < dimsrc; ++i) {
      dst_in_src_stride_[i] = step[axes[i]];
      this->shape_[i] = sshape[axes[i]];
    }
  }
};
template <typename SrcExp, typename DType, int etype>
inline TransposeExExp<SrcExp, DType, ExpInfo<SrcExp>::kDim> transpose(
    const Exp<SrcExp, DType, etype> &src, Shape<ExpInfo<SrcExp>::kDim> axes) {
  return TransposeExExp<SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), axes);
}
template <typename SrcExp, typename DType, int dimsrc>
struct Plan<TransposeExExp<SrcExp, DType, dimsrc>, DType> {
 public:
  explicit Plan(const TransposeExExp<SrcExp, DType, dimsrc> &e)
      : src_(MakePlan(e.src_)), at_(e.src_stride_), step_(e.dst_in_src_stride_),
        digits_(e.shape_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    index_t flat = j * step_[dimsrc - 1];
#pragma unroll
    for (int k = dimsrc - 2; k >= 0; --k) flat += digits_.Pop(k, i) * step_[k];
    return at_.Eval(src_, flat);
  }
  /* a permutation that leaves the last axis in place permutes rows */
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t i, index_t j) const {
    index_t flat = 0;
#pragma unroll
    for (int k = dimsrc - 2; k >= 0; --k) flat += digits_.Pop(k, i) * step_[k];
    return src_.template EvalPack<N, STREAM>(at_.last.Div(flat), j);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    return axes_detail::SourcePackReady(src_, n, cols, flat) && step_[dimsrc - 1] == 1;
  }

 private:
  Plan<SrcExp, DType> src_;
  const axes_detail::FlatAt at_;
  const Shape<dimsrc> step_;
  const axes_detail::RowDigits<dimsrc> digits_;
};

/*! \brief flat indices into a tensor of shape src_shape mapped to the flat indices of the same
 *  elements after transpose(axes) */
template <typename SrcExp, typename DType, int dimsrc, int etype>
struct TransposeIndicesExp : public Exp<TransposeIndicesExp<SrcExp, DType, dimsrc, etype>, DType,
                                        etype> {
  const SrcExp &src_indices_;
  Shape<dimsrc> src_shape_;
  const Shape<dimsrc> axes_;
  Shape<dimsrc> src_in_dst_stride_;  //!< distance in the result of a step along each source axis
  TransposeIndicesExp(const SrcExp &src_indices, Shape<dimsrc> src_shape, Shape<dimsrc> axes)
      : src_indices_(src_indices), src_shape_(src_shape), axes_(axes) {
    Shape<dimsrc> dshape, dstep;
    bool seen[dimsrc] = {0};
    for (int i = 0; i < dimsrc; ++i) {
      CHECK_LT(static_cast<int>(axes[i]), dimsrc)
          << "Invalid axes input! All elements of axes must be between 0 and " << dimsrc
          << ", find axes=" << axes;
      dshape[i] = src_shape[axes[i]];
      seen[axes[i]] = true;
    }
    for (int i = 0; i < dimsrc; ++i) {
      CHECK_EQ(seen[i], true) << "Invalid axes input! All elements of axes must be between 0 and "
                              << dimsrc << ", find axes=" << axes;
    }
    dstep[dimsrc - 1] = 1;
    for (int i = dimsrc - 2; i >= 0; --i) dstep[i] = dshape[i + 1] * dstep[i + 1];
    for (int i = 0; i < dimsrc; ++i) src_in_dst_stride_[axes[i]] = dstep[i];
  }
};
template <typename SrcExp, typename DType, int dimsrc, int etype>
inline TransposeIndicesExp<SrcExp, DType, dimsrc, etype> transpose_indices(
    const Exp<SrcExp, DType, etype> &src_indices, Shape<dimsrc> src_shape, Shape<dimsrc> axes) {
  return TransposeIndicesExp<SrcExp, DType, dimsrc, etype>(src_indices.self(), src_shape, axes);
}
template <typename SrcExp, typename DType, int dimsrc, int etype>
struct Plan<TransposeIndicesExp<SrcExp, DType, dimsrc, etype>, DType> {
 public:
  explicit Plan(const TransposeIndicesExp<SrcExp, DType, dimsrc, etype> &e)
      : src_indices_(MakePlan(e.src_indices_)), step_(e.src_in_dst_stride_) {
    for (int k = 0; k < dimsrc; ++k) len_[k] = FastDivU32(e.src_shape_[k]);
  }
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    index_t rest = static_cast<index_t>(src_indices_.Eval(i, j));
    index_t dst = 0;
#pragma unroll
    for (int k = dimsrc - 1; k >= 0; --k) {
      const index_t q = len_[k].Div(rest);
      dst += (rest - q * len_[k].div) * step_[k];
      rest = q;
    }
    return static_cast<DType>(dst);
  }

 private:
  Plan<SrcExp, DType> src_indices_;
  const Shape<dimsrc> step_;
  FastDivU32 len_[dimsrc];
};
template <typename SrcExp, typename DType, int dimsrc, int etype>
inline Plan<TransposeIndicesExp<SrcExp, DType, dimsrc, etype>, DType> MakePlan(
    const TransposeIndicesExp<SrcExp, DType, dimsrc, etype> &e) {
  return Plan<TransposeIndicesExp<SrcExp, DType, dimsrc, etype>, DType>(e);
}
template <int dim, typename SrcExp, typename DType, int dimsrc, int etype>
struct ShapeCheck<dim, TransposeIndicesExp<SrcExp, DType, dimsrc, etype> > {
  inline static Shape<dim> Check(const TransposeIndicesExp<SrcExp, DType, dimsrc, etype> &t) {
    return ShapeCheck<dim, SrcExp>::Check(t.src_indices_);
  }
};
template <typename SrcExp, typename DType, int dimsrc, int etype>
struct ExpInfo<TransposeIndicesExp<SrcExp, DType, dimsrc, etype> > {
  static const int kDim = ExpInfo<SrcExp>::kDim;
  static const int kDevMask = ExpInfo<SrcExp>::kDevMask;
};

/* ------------------------------------------------------------------ views that can be assigned to
 * ConcatExp, SliceExp, SliceExExp and FlipExp are TRValues: `slice<1>(t, 2, 5) = expr` and
 * `concat<1>(a, b) = expr` write through REval. */
#define MSHADOW_VIEW_ASSIGN                                                    \
  template <typename E, int etype>                                             \
  inline void operator=(const expr::Exp<E, DType, etype> &exp) {               \
    this->__assign(exp);                                                       \
  }                                                                            \
  inline void operator=(const DType &exp) { this->__assign(exp); }

/*! \brief two expressions side by side along dimension srcdim - dimsrc_m_cat */
template <typename LhsExp, typename RhsExp, typename Device, typename DType, int srcdim,
          int dimsrc_m_cat>
struct ConcatExp : public TRValue<ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, dimsrc_m_cat>,
                                  Device, srcdim, DType> {
  static const int dimcat = srcdim - dimsrc_m_cat;
  const LhsExp &src1_;
  const RhsExp &src2_;
  index_t dcat_src1_, dcat_src2_;
  Shape<srcdim> shape_;
  ConcatExp(const LhsExp &src1, const RhsExp &src2) : src1_(src1), src2_(src2) {
    Shape<srcdim> s1 = ShapeCheck<srcdim, LhsExp>::Check(src1_);
    Shape<srcdim> s2 = ShapeCheck<srcdim, RhsExp>::Check(src2_);
    for (int i = 0; i < srcdim; ++i) {
      if (i != dimcat) CHECK_EQ(s1[i], s2[i]) << "ConcatExp: shape mismatch";
    }
    shape_ = s1;
    shape_[dimcat] = s1[dimcat] + s2[dimcat];
    dcat_src1_ = s1[dimcat];
    dcat_src2_ = s2[dimcat];
  }
  MSHADOW_VIEW_ASSIGN
};
template <int cdim, typename LhsExp, typename RhsExp, typename Device, typename DType, int srcdim>
inline ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, srcdim - cdim> concat(
    const TRValue<LhsExp, Device, srcdim, DType> &src1,
    const TRValue<RhsExp, Device, srcdim, DType> &src2) {
  TypeCheckPass<ExpInfo<LhsExp>::kDim == ExpInfo<RhsExp>::kDim>::
      Error_Expression_Does_Not_Meet_Dimension_Req();
  TypeCheckPass<(cdim < srcdim) && ExpInfo<LhsExp>::kDim == srcdim>::
      Error_Expression_Does_Not_Meet_Dimension_Req();
  return ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, srcdim - cdim>(src1.self(), src2.self());
}
template <typename LhsExp, typename RhsExp, typename Device, typename DType, int srcdim,
          int dimsrc_m_cat>
struct ShapeCheck<srcdim, ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, dimsrc_m_cat> > {
  inline static Shape<srcdim> Check(
      const ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, dimsrc_m_cat> &t) {
    return t.shape_;
  }
};
template <typename LhsExp, typename RhsExp, typename Device, typename DType, int srcdim,
          int dimsrc_m_cat>
struct StreamInfo<Device, ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, dimsrc_m_cat> > {
  inline static Stream<Device> *Get(
      const ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, dimsrc_m_cat> &t) {
    Stream<Device> *lhs = StreamInfo<Device, LhsExp>::Get(t.src1_);
    Stream<Device> *rhs = StreamInfo<Device, RhsExp>::Get(t.src2_);
    return lhs == rhs ? lhs : NULL;
  }
};
template <typename LhsExp, typename RhsExp, typename Device, typename DType, int srcdim,
          int dimsrc_m_cat>
struct ExpInfo<ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, dimsrc_m_cat> > {
  static const int kDimLhs = ExpInfo<LhsExp>::kDim;
  static const int kDimRhs = ExpInfo<RhsExp>::kDim;
  static const int kDim =
      (kDimLhs < 0 || kDimRhs < 0) ? -1
      : (kDimLhs == 0)             ? kDimRhs
      : (kDimRhs == 0 || kDimLhs == kDimRhs) ? kDimLhs : -1;
  static const int kDevMask = ExpInfo<LhsExp>::kDevMask & ExpInfo<RhsExp>::kDevMask;
};
/* concatenation along a leading dimension: its index is a digit of the row number */
template <typename LhsExp, typename RhsExp, typename Device, typename DType, int srcdim,
          int dimsrc_m_cat>
struct Plan<ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, dimsrc_m_cat>, DType> {
 public:
  static const int dimcat = srcdim - dimsrc_m_cat;
  explicit Plan(const ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, dimsrc_m_cat> &e)
      : src1_(MakePlan(e.src1_)), src2_(MakePlan(e.src2_)),
        height_(e.shape_.ProdShape(dimcat + 1, srcdim - 1)), ch_(e.shape_[dimcat]),
        ch_src1_(e.dcat_src1_), ch_src2_(e.dcat_src2_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    bool second;
    const index_t row = Locate(i, &second);
    return second ? src2_.Eval(row, j) : src1_.Eval(row, j);
  }
  MSHADOW_XINLINE DType &REval(index_t i, index_t j) {
    bool second;
    const index_t row = Locate(i, &second);
    return second ? src2_.REval(row, j) : src1_.REval(row, j);
  }
  static const bool kPackable = plan_detail::Packable<Plan<LhsExp, DType> >::value &&
                                plan_detail::Packable<Plan<RhsExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t i, index_t j) const {
    bool second;
    const index_t row = Locate(i, &second);
    return second ? src2_.template EvalPack<N, STREAM>(row, j)
                  : src1_.template EvalPack<N, STREAM>(row, j);
  }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE void StorePack(index_t i, index_t j, const Pack<DType, N> &p) {
    bool second;
    const index_t row = Locate(i, &second);
    if (second) src2_.template StorePack<N, STREAM>(row, j, p);
    else src1_.template StorePack<N, STREAM>(row, j, p);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    return axes_detail::SourcePackReady(src1_, n, cols, flat) &&
           axes_detail::SourcePackReady(src2_, n, cols, flat);
  }

 private:
  /*! \brief which operand holds row i of the concatenation, and at which of its rows */
  MSHADOW_XINLINE index_t Locate(index_t i, bool *second) const {
    const index_t upper = height_.Div(i);
    const index_t y = i - upper * height_.div;
    const index_t b = ch_.Div(upper);
    const index_t c = upper - b * ch_.div;
    *second = c >= ch_src1_;
    return *second ? (b * ch_src2_ + c - ch_src1_) * height_.div + y
                   : (b * ch_src1_ + c) * height_.div + y;
  }
  Plan<LhsExp, DType> src1_;
  Plan<RhsExp, DType> src2_;
  const FastDivU32 height_, ch_;
  const index_t ch_src1_, ch_src2_;
};
/* concatenation along the last dimension: a column offset */
template <typename LhsExp, typename RhsExp, typename Device, typename DType, int srcdim>
struct Plan<ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, 1>, DType> {
 public:
  explicit Plan(const ConcatExp<LhsExp, RhsExp, Device, DType, srcdim, 1> &e)
      : src1_(MakePlan(e.src1_)), src2_(MakePlan(e.src2_)), width_src1_(e.dcat_src1_) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    return x < width_src1_ ? src1_.Eval(y, x) : src2_.Eval(y, x - width_src1_);
  }
  MSHADOW_XINLINE DType &REval(index_t y, index_t x) {
    return x < width_src1_ ? src1_.REval(y, x) : src2_.REval(y, x - width_src1_);
  }

 private:
  Plan<LhsExp, DType> src1_;
  Plan<RhsExp, DType> src2_;
  const index_t width_src1_;
};

/*! \brief positions [begin, end) of dimension srcdim - dimsrc_m_slice */
template <typename SrcExp, typename Device, typename DType, int srcdim, int dimsrc_m_slice>
struct SliceExp : public TRValue<SliceExp<SrcExp, Device, DType, srcdim, dimsrc_m_slice>, Device,
                                 srcdim, DType> {
  static const int dimslice = srcdim - dimsrc_m_slice;
  const SrcExp &src_;
  index_t ch_begin_, ch_old_;
  Shape<srcdim> shape_;
  SliceExp(const SrcExp &src, index_t begin, index_t end) : src_(src), ch_begin_(begin) {
    shape_ = ShapeCheck<srcdim, SrcExp>::Check(src_);
    ch_old_ = shape_[dimslice];
    CHECK(begin < shape_[dimslice] && end <= shape_[dimslice]) << "The slice went out of range";
    shape_[dimslice] = end - begin;
  }
  MSHADOW_VIEW_ASSIGN
};
template <int sdim, typename SrcExp, typename Device, typename DType, int srcdim>
inline SliceExp<SrcExp, Device, DType, srcdim, srcdim - sdim> slice(
    const TRValue<SrcExp, Device, srcdim, DType> &src, index_t begin, index_t end) {
  TypeCheckPass<(sdim < srcdim) && ExpInfo<SrcExp>::kDim == srcdim>::
      Error_Expression_Does_Not_Meet_Dimension_Req();
  return SliceExp<SrcExp, Device, DType, srcdim, srcdim - sdim>(src.self(), begin, end);
}
template <typename SrcExp, typename Device, typename DType, int srcdim, int dimsrc_m_slice>
struct ShapeCheck<srcdim, SliceExp<SrcExp, Device, DType, srcdim, dimsrc_m_slice> > {
  inline static Shape<srcdim> Check(
      const SliceExp<SrcExp, Device, DType, srcdim, dimsrc_m_slice> &t) {
    return t.shape_;
  }
};
template <typename SrcExp, typename Device, typename DType, int srcdim, int dimsrc_m_slice>
struct StreamInfo<Device, SliceExp<SrcExp, Device, DType, srcdim, dimsrc_m_slice> > {
  inline static Stream<Device> *Get(
      const SliceExp<SrcExp, Device, DType, srcdim, dimsrc_m_slice> &t) {
    return StreamInfo<Device, SrcExp>::Get(t.src_);
  }
};
template <typename SrcExp, typename Device, typename DType, int srcdim, int dimsrc_m_slice>
struct ExpInfo<SliceExp<SrcExp, Device, DType, srcdim, dimsrc_m_slice> > {
  static const int kDim = ExpInfo<SrcExp>::kDim;
  static const int kDevMask = ExpInfo<SrcExp>::kDevMask;
};
template <typename SrcExp, typename Device, typename DType, int srcdim, int dimsrc_m_slice>
struct Plan<SliceExp<SrcExp, Device, DType, srcdim, dimsrc_m_slice>, DType> {
 public:
  static const int dimslice = srcdim - dimsrc_m_slice;
  explicit Plan(const SliceExp<SrcExp, Device, DType, srcdim, dimsrc_m_slice> &e)
      : src_(MakePlan(e.src_)), height_(e.shape_.ProdShape(dimslice + 1, srcdim - 1)),
        ch_(e.shape_[dimslice]), ch_begin_(e.ch_begin_), ch_old_(e.ch_old_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const { return src_.Eval(Row(i), j); }
  MSHADOW_XINLINE DType &REval(index_t i, index_t j) { return src_.REval(Row(i), j); }
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t i, index_t j) const {
    return src_.template EvalPack<N, STREAM>(Row(i), j);
  }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE void StorePack(index_t i, index_t j, const Pack<DType, N> &p) {
    src_.template StorePack<N, STREAM>(Row(i), j, p);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    return axes_detail::SourcePackReady(src_, n, cols, flat);
  }

 private:
  MSHADOW_XINLINE index_t Row(index_t i) const {
    const index_t upper = height_.Div(i);
    const index_t y = i - upper * height_.div;
    const index_t b = ch_.Div(upper);
    const index_t c = upper - b * ch_.div + ch_begin_;
    return (b * ch_old_ + c) * height_.div + y;
  }
  Plan<SrcExp, DType> src_;
  const FastDivU32 height_, ch_;
  const index_t ch_begin_, ch_old_;
};
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct Plan<SliceExp<SrcExp, Device, DType, srcdim, 1>, DType> {
 public:
  explicit Plan(const SliceExp<SrcExp, Device, DType, srcdim, 1> &e)
      : src_(MakePlan(e.src_)), ch_begin_(e.ch_begin_) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const { return src_.Eval(y, x + ch_begin_); }
  MSHADOW_XINLINE DType &REval(index_t y, index_t x) { return src_.REval(y, x + ch_begin_); }

 private:
  Plan<SrcExp, DType> src_;
  const index_t ch_begin_;
};

/*! \brief positions [begin[k], end[k]) of every dimension k */
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct SliceExExp
    : public TRValue<SliceExExp<SrcExp, Device, DType, srcdim>, Device, srcdim, DType> {
  const SrcExp &src_;
  Shape<srcdim> src_shape_;
  Shape<srcdim> shape_;
  const Shape<srcdim> begin_, end_;
  SliceExExp(const SrcExp &src, Shape<srcdim> begin, Shape<srcdim> end)
      : src_(src), begin_(begin), end_(end) {
    src_shape_ = ShapeCheck<srcdim, SrcExp>::Check(src_);
    for (int i = 0; i < srcdim; ++i) shape_[i] = end_[i] - begin_[i];
  }
  MSHADOW_VIEW_ASSIGN
};
template <typename SrcExp, typename Device, typename DType, int srcdim>
inline SliceExExp<SrcExp, Device, DType, srcdim> slice(
    const TRValue<SrcExp, Device, srcdim, DType> &src, Shape<srcdim> begin, Shape<srcdim> end) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim == srcdim>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return SliceExExp<SrcExp, Device, DType, srcdim>(src.self(), begin, end);
}
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct ShapeCheck<srcdim, SliceExExp<SrcExp, Device, DType, srcdim> > {
  inline static Shape<srcdim> Check(const SliceExExp<SrcExp, Device, DType, srcdim> &t) {
    return t.shape_;
  }
};
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct StreamInfo<Device, SliceExExp<SrcExp, Device, DType, srcdim> > {
  inline static Stream<Device> *Get(const SliceExExp<SrcExp, Device, DType, srcdim> &t) {
    return StreamInfo<Device, SrcExp>::Get(t.src_);
  }
};
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct ExpInfo<SliceExExp<SrcExp, Device, DType, srcdim> > {
  static const int kDim = ExpInfo<SrcExp>::kDim;
  static const int kDevMask = ExpInfo<SrcExp>::kDevMask;
};
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct Plan<SliceExExp<SrcExp, Device, DType, srcdim>, DType> {
 public:
  explicit Plan(const SliceExExp<SrcExp, Device, DType, srcdim> &e)
      : src_(MakePlan(e.src_)), begin_(e.begin_), src_shape_(e.src_shape_), digits_(e.shape_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    return src_.Eval(Row(i), j + begin_[srcdim - 1]);
  }
  MSHADOW_XINLINE DType &REval(index_t i, index_t j) {
    return src_.REval(Row(i), j + begin_[srcdim - 1]);
  }

 private:
  MSHADOW_XINLINE index_t Row(index_t i) const {
    index_t row = 0, step = 1;
#pragma unroll
    for (int k = srcdim - 2; k >= 0; --k) {
      row += step * (digits_.Pop(k, i) + begin_[k]);
      step *= src_shape_[k];
    }
    return row;
  }
  Plan<SrcExp, DType> src_;
  const Shape<srcdim> begin_, src_shape_;
  const axes_detail::RowDigits<srcdim> digits_;
};

/*! \brief dimension `dim` reversed */
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct FlipExp : public TRValue<FlipExp<SrcExp, Device, DType, srcdim>, Device, srcdim, DType> {
  const SrcExp &src_;
  index_t trailing_;  //!< elements spanned by the dimensions after `dim`
  index_t stride_;    //!< length of `dim`
  index_t stride_j_;  //!< last dimension
  Shape<srcdim> shape_;
  FlipExp(const SrcExp &src, int dim) : src_(src) {
    shape_ = ShapeCheck<srcdim, SrcExp>::Check(src_);
    stride_ = shape_[dim];
    stride_j_ = shape_[srcdim - 1];
    trailing_ = 1;
    for (int i = dim + 1; i < srcdim; ++i) trailing_ *= shape_[i];
  }
  MSHADOW_VIEW_ASSIGN
};
template <typename SrcExp, typename Device, typename DType, int srcdim>
inline FlipExp<SrcExp, Device, DType, srcdim> flip(const TRValue<SrcExp, Device, srcdim, DType> &src,
                                                  int dim) {
  return FlipExp<SrcExp, Device, DType, srcdim>(src.self(), dim);
}
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct ShapeCheck<srcdim, FlipExp<SrcExp, Device, DType, srcdim> > {
  inline static Shape<srcdim> Check(const FlipExp<SrcExp, Device, DType, srcdim> &t) {
    return t.shape_;
  }
};
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct StreamInfo<Device, FlipExp<SrcExp, Device, DType, srcdim> > {
  inline static Stream<Device> *Get(const FlipExp<SrcExp, Device, DType, srcdim> &t) {
    return StreamInfo<Device, SrcExp>::Get(t.src_);
  }
};
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct ExpInfo<FlipExp<SrcExp, Device, DType, srcdim> > {
  static const int kDim = ExpInfo<SrcExp>::kDim;
  static const int kDevMask = ExpInfo<SrcExp>::kDevMask;
};
template <typename SrcExp, typename Device, typename DType, int srcdim>
struct Plan<FlipExp<SrcExp, Device, DType, srcdim>, DType> {
 public:
  explicit Plan(const FlipExp<SrcExp, Device, DType, srcdim> &e)
      : src_(MakePlan(e.src_)), at_(e.stride_j_), trailing_(e.trailing_), stride_(e.stride_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const { return at_.Eval(src_, Mirror(i, j)); }
  MSHADOW_XINLINE DType &REval(index_t i, index_t j) { return at_.REval(src_, Mirror(i, j)); }
  /* reversing any axis but the last reverses runs of whole rows */
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t i, index_t j) const {
    return src_.template EvalPack<N, STREAM>(at_.last.Div(Mirror(i, 0)), j);
  }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE void StorePack(index_t i, index_t j, const Pack<DType, N> &p) {
    src_.template StorePack<N, STREAM>(at_.last.Div(Mirror(i, 0)), j, p);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    return axes_detail::SourcePackReady(src_, n, cols, flat) &&
           trailing_.div % at_.last.div == 0;
  }

 private:
  MSHADOW_XINLINE index_t Mirror(index_t i, index_t j) const {
    const index_t flat = i * at_.last.div + j;
    const index_t upper = trailing_.Div(flat);
    const index_t low = flat - upper * trailing_.div;
    const index_t high = stride_.Div(upper);
    const index_t x = upper - high * stride_.div;
    return (high * stride_.div + stride_.div - 1 - x) * trailing_.div + low;
  }
  Plan<SrcExp, DType> src_;
  const axes_detail::FlatAt at_;
  const FastDivU32 trailing_, stride_;
};
#undef MSHADOW_VIEW_ASSIGN

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_AXES_H_
