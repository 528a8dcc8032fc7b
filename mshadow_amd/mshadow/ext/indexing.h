/*
 * Expression nodes that look rows or elements up by an index vector:
 *   take(index, src)                        out[y][x] = src[index[y]][x]
 *   take_grad(index, src, input_dim)        out[y][x] = sum over i with index[i] == y of src[i][x]
 *   one_hot_encode(index, num_choices)      out[y][x] = (x == index[y])
 *   mat_choose_row_element(src, index)      out[x]    = src[x][index[x]]
 *   mat_fill_row_element(src, val, index)   out[y][x] = x == index[y] ? val[y] : src[y][x]
 *   mask(index, src)                        out[y][x] = src[y][x] * index[y]
 *   range(start, stop, step, repeat)        out[x]    = start + (x / repeat) * step
 *
 * Semantics restate the reference's nodes of the same names (mshadow/extension/take.h:14-97,
 * take_grad.h:14-107, one_hot.h:14-87, choose.h:14-90, fill.h:14-103, mask.h:14-97,
 * range.h:14-118). Indices travel as values of the element type and are converted with
 * static_cast<index_t>; nothing checks them against the source's extent. take_grad adds the
 * matching rows in ascending i into a zero.
 */
#ifndef MSHADOW_EXT_INDEXING_H_
#define MSHADOW_EXT_INDEXING_H_

#include <cmath>

#include "../tensor.h"

namespace mshadow {
namespace expr {

/* the nodes below are chainers that do not go through MakeTensorExp: their shape is derived
   from two operands when it is asked for, so each brings its own MakePlan / ShapeCheck /
   ExpInfo */

/* ------------------------------------------------------------------ take */
template <typename IndexExp, typename SrcExp, typename DType>
struct TakeExp : public Exp<TakeExp<IndexExp, SrcExp, DType>, DType, type::kChainer> {
  const IndexExp &index_;
  const SrcExp &src_;
  TakeExp(const IndexExp &index, const SrcExp &src) : index_(index), src_(src) {}
};
template <typename IndexExp, typename SrcExp, typename DType, int e1, int e2>
inline TakeExp<IndexExp, SrcExp, DType> take(const Exp<IndexExp, DType, e1> &index,
                                             const Exp<SrcExp, DType, e2> &src) {
  return TakeExp<IndexExp, SrcExp, DType>(index.self(), src.self());
}
template <typename IndexExp, typename SrcExp, typename DType>
struct Plan<TakeExp<IndexExp, SrcExp, DType>, DType> {
 public:
  explicit Plan(const TakeExp<IndexExp, SrcExp, DType> &e)
      : index_(MakePlan(e.index_)), src_(MakePlan(e.src_)) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    return static_cast<DType>(src_.Eval(static_cast<index_t>(index_.Eval(0, y)), x));
  }
  /* a row of the result is a row of the source */
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    return src_.template EvalPack<N, false>(static_cast<index_t>(index_.Eval(0, y)), x);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    *flat = false;
    bool ignored = true;
    return src_.PackReady(n, cols, &ignored);
  }

 private:
  Plan<IndexExp, DType> index_;
  Plan<SrcExp, DType> src_;
};
template <typename IndexExp, typename SrcExp, typename DType>
inline Plan<TakeExp<IndexExp, SrcExp, DType>, DType> MakePlan(
    const TakeExp<IndexExp, SrcExp, DType> &exp) {
  return Plan<TakeExp<IndexExp, SrcExp, DType>, DType>(exp);
}
template <int dim, typename IndexExp, typename SrcExp, typename DType>
struct ShapeCheck<dim, TakeExp<IndexExp, SrcExp, DType> > {
  inline static Shape<dim> Check(const TakeExp<IndexExp, SrcExp, DType> &t) {
    CHECK(dim == 2) << "TakeExp only support 2D output";
    Shape<1> ishape = ShapeCheck<1, IndexExp>::Check(t.index_);
    Shape<2> sshape = ShapeCheck<2, SrcExp>::Check(t.src_);
    Shape<dim> ret;
    ret[0] = ishape[0];
    ret[1] = sshape[1];
    return ret;
  }
};
template <typename IndexExp, typename SrcExp, typename DType>
struct ExpInfo<TakeExp<IndexExp, SrcExp, DType> > {
  static const int kDim = 2;
  static const int kDevMask = ExpInfo<IndexExp>::kDevMask;
};

/* ------------------------------------------------------------------ take_grad */
template <typename IndexExp, typename SrcExp, typename DType>
struct TakeGradExp : public Exp<TakeGradExp<IndexExp, SrcExp, DType>, DType, type::kChainer> {
  const IndexExp &index_;
  const SrcExp &src_;
  const index_t input_dim_;
  TakeGradExp(const IndexExp &index, const SrcExp &src, const index_t input_dim)
      : index_(index), src_(src), input_dim_(input_dim) {}
};
template <typename IndexExp, typename SrcExp, typename DType, int e1, int e2>
inline TakeGradExp<IndexExp, SrcExp, DType> take_grad(const Exp<IndexExp, DType, e1> &index,
                                                      const Exp<SrcExp, DType, e2> &src,
                                                      const index_t input_dim) {
  return TakeGradExp<IndexExp, SrcExp, DType>(index.self(), src.self(), input_dim);
}
template <typename IndexExp, typename SrcExp, typename DType>
struct Plan<TakeGradExp<IndexExp, SrcExp, DType>, DType> {
 public:
  explicit Plan(const TakeGradExp<IndexExp, SrcExp, DType> &e)
      : index_(MakePlan(e.index_)), src_(MakePlan(e.src_)),
        batch_size_(ShapeCheck<1, IndexExp>::Check(e.index_)[0]) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    DType ret = 0.f;
    for (index_t i = 0; i < batch_size_; ++i) {
      if (static_cast<index_t>(index_.Eval(0, i)) == y) ret += static_cast<DType>(src_.Eval(i, x));
    }
    return ret;
  }

 private:
  Plan<IndexExp, DType> index_;
  Plan<SrcExp, DType> src_;
  const index_t batch_size_;
};
template <typename IndexExp, typename SrcExp, typename DType>
inline Plan<TakeGradExp<IndexExp, SrcExp, DType>, DType> MakePlan(
    const TakeGradExp<IndexExp, SrcExp, DType> &exp) {
  return Plan<TakeGradExp<IndexExp, SrcExp, DType>, DType>(exp);
}
template <int dim, typename IndexExp, typename SrcExp, typename DType>
struct ShapeCheck<dim, TakeGradExp<IndexExp, SrcExp, DType> > {
  inline static Shape<dim> Check(const TakeGradExp<IndexExp, SrcExp, DType> &t) {
    CHECK(dim == 2) << "TakeGradExp only support 2D output";
    Shape<2> gshape = ShapeCheck<2, SrcExp>::Check(t.src_);
    Shape<dim> ret;
    ret[0] = t.input_dim_;
    ret[1] = gshape[1];
    return ret;
  }
};
template <typename IndexExp, typename SrcExp, typename DType>
struct ExpInfo<TakeGradExp<IndexExp, SrcExp, DType> > {
  static const int kDim = 2;
  static const int kDevMask = ExpInfo<IndexExp>::kDevMask;
};

/* ------------------------------------------------------------------ mask */
template <typename IndexExp, typename SrcExp, typename DType>
struct MaskExp : public Exp<MaskExp<IndexExp, SrcExp, DType>, DType, type::kChainer> {
  const IndexExp &index_;
  const SrcExp &src_;
  MaskExp(const IndexExp &index, const SrcExp &src) : index_(index), src_(src) {}
};
template <typename IndexExp, typename SrcExp, typename DType, int e1, int e2>
inline MaskExp<IndexExp, SrcExp, DType> mask(const Exp<IndexExp, DType, e1> &index,
                                             const Exp<SrcExp, DType, e2> &src) {
  return MaskExp<IndexExp, SrcExp, DType>(index.self(), src.self());
}
template <typename IndexExp, typename SrcExp, typename DType>
struct Plan<MaskExp<IndexExp, SrcExp, DType>, DType> {
 public:
  explicit Plan(const MaskExp<IndexExp, SrcExp, DType> &e)
      : index_(MakePlan(e.index_)), src_(MakePlan(e.src_)) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    return static_cast<DType>(src_.Eval(y, x) * index_.Eval(0, y));
  }
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    Pack<DType, N> p = src_.template EvalPack<N, STREAM>(y, x);
    const DType factor = index_.Eval(0, y);
#pragma unroll
    for (int k = 0; k < N; ++k) p.v[k] = static_cast<DType>(p.v[k] * factor);
    return p;
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    *flat = false;
    bool ignored = true;
    return src_.PackReady(n, cols, &ignored);
  }

 private:
  Plan<IndexExp, DType> index_;
  Plan<SrcExp, DType> src_;
};
template <typename IndexExp, typename SrcExp, typename DType>
inline Plan<MaskExp<IndexExp, SrcExp, DType>, DType> MakePlan(
    const MaskExp<IndexExp, SrcExp, DType> &exp) {
  return Plan<MaskExp<IndexExp, SrcExp, DType>, DType>(exp);
}
template <int dim, typename IndexExp, typename SrcExp, typename DType>
struct ShapeCheck<dim, MaskExp<IndexExp, SrcExp, DType> > {
  inline static Shape<dim> Check(const MaskExp<IndexExp, SrcExp, DType> &t) {
    CHECK(dim == 2) << "MaskExp only support 2D output";
    Shape<1> ishape = ShapeCheck<1, IndexExp>::Check(t.index_);
    Shape<2> sshape = ShapeCheck<2, SrcExp>::Check(t.src_);
    CHECK_EQ(ishape[0], sshape[0]) << "MaskExp require inputs in same first dimention";
    Shape<dim> ret;
    ret[0] = sshape[0];
    ret[1] = sshape[1];
    return ret;
  }
};
template <typename IndexExp, typename SrcExp, typename DType>
struct ExpInfo<MaskExp<IndexExp, SrcExp, DType> > {
  static const int kDim = 2;
  static const int kDevMask = ExpInfo<IndexExp>::kDevMask;
};

/* ------------------------------------------------------------------ one_hot_encode */
template <typename IndexExp, typename DType>
struct OneHotEncodeExp : public Exp<OneHotEncodeExp<IndexExp, DType>, DType, type::kChainer> {
  const IndexExp &index_;
  index_t num_choices_;
  OneHotEncodeExp(const IndexExp &index, index_t num_choices)
      : index_(index), num_choices_(num_choices) {}
};
/*! \brief the result's element type is default_real_t whatever the index's */
template <typename IndexExp, typename IDType, int e1>
inline OneHotEncodeExp<IndexExp, default_real_t> one_hot_encode(
    const Exp<IndexExp, IDType, e1> &index, index_t num_choices) {
  TypeCheckPass<ExpInfo<IndexExp>::kDim == 1>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return OneHotEncodeExp<IndexExp, default_real_t>(index.self(), num_choices);
}
template <typename IndexExp, typename DType>
struct Plan<OneHotEncodeExp<IndexExp, DType>, DType> {
 public:
  explicit Plan(const OneHotEncodeExp<IndexExp, DType> &e) : index_(MakePlan(e.index_)) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    return static_cast<DType>(x == static_cast<index_t>(index_.Eval(0, y)));
  }

 private:
  Plan<IndexExp, DType> index_;
};
template <typename IndexExp, typename DType>
inline Plan<OneHotEncodeExp<IndexExp, DType>, DType> MakePlan(
    const OneHotEncodeExp<IndexExp, DType> &exp) {
  return Plan<OneHotEncodeExp<IndexExp, DType>, DType>(exp);
}
template <int dim, typename IndexExp, typename DType>
struct ShapeCheck<dim, OneHotEncodeExp<IndexExp, DType> > {
  inline static Shape<dim> Check(const OneHotEncodeExp<IndexExp, DType> &t) {
    CHECK(dim == 2) << "OneHotEncodeExp only support 2 dimension output";
    Shape<1> ishape = ShapeCheck<1, IndexExp>::Check(t.index_);
    Shape<dim> ret;
    ret[0] = ishape[0];
    ret[1] = t.num_choices_;
    return ret;
  }
};
template <typename IndexExp, typename DType>
struct ExpInfo<OneHotEncodeExp<IndexExp, DType> > {
  static const int kDim = 2;
  static const int kDevMask = ExpInfo<IndexExp>::kDevMask;
};

/* ------------------------------------------------------------------ mat_choose_row_element */
template <typename SrcExp, typename IndexExp, typename DType>
struct MatChooseRowElementExp
    : public Exp<MatChooseRowElementExp<SrcExp, IndexExp, DType>, DType, type::kChainer> {
  const SrcExp &src_;
  const IndexExp &index_;
  MatChooseRowElementExp(const SrcExp &src, const IndexExp &index) : src_(src), index_(index) {}
};
template <typename SrcExp, typename IndexExp, typename DType, typename IDType, int e1, int e2>
inline MatChooseRowElementExp<SrcExp, IndexExp, DType> mat_choose_row_element(
    const Exp<SrcExp, DType, e1> &src, const Exp<IndexExp, IDType, e2> &index) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim == 2 && ExpInfo<IndexExp>::kDim == 1>::
      Error_Expression_Does_Not_Meet_Dimension_Req();
  return MatChooseRowElementExp<SrcExp, IndexExp, DType>(src.self(), index.self());
}
template <typename SrcExp, typename IndexExp, typename DType>
struct Plan<MatChooseRowElementExp<SrcExp, IndexExp, DType>, DType> {
 public:
  explicit Plan(const MatChooseRowElementExp<SrcExp, IndexExp, DType> &e)
      : src_(MakePlan(e.src_)), index_(MakePlan(e.index_)) {}
  MSHADOW_XINLINE DType Eval(index_t, index_t x) const {
    return src_.Eval(x, static_cast<index_t>(index_.Eval(0, x)));
  }

 private:
  Plan<SrcExp, DType> src_;
  Plan<IndexExp, DType> index_;
};
template <typename SrcExp, typename IndexExp, typename DType>
inline Plan<MatChooseRowElementExp<SrcExp, IndexExp, DType>, DType> MakePlan(
    const MatChooseRowElementExp<SrcExp, IndexExp, DType> &exp) {
  return Plan<MatChooseRowElementExp<SrcExp, IndexExp, DType>, DType>(exp);
}
template <int dim, typename SrcExp, typename IndexExp, typename DType>
struct ShapeCheck<dim, MatChooseRowElementExp<SrcExp, IndexExp, DType> > {
  inline static Shape<dim> Check(const MatChooseRowElementExp<SrcExp, IndexExp, DType> &t) {
    CHECK(dim == 1) << "MatChooseRowElementExp only support 1 dimension output";
    Shape<2> sshape = ShapeCheck<2, SrcExp>::Check(t.src_);
    Shape<dim> ishape = ShapeCheck<dim, IndexExp>::Check(t.index_);
    CHECK_EQ(sshape[0], ishape[0])
        << "mat_choose_row_element index length and number of rows in matrix";
    return ishape;
  }
};
template <typename SrcExp, typename IndexExp, typename DType>
struct ExpInfo<MatChooseRowElementExp<SrcExp, IndexExp, DType> > {
  static const int kDim = 1;
  static const int kDevMask = ExpInfo<SrcExp>::kDevMask & ExpInfo<IndexExp>::kDevMask;
};

/* ------------------------------------------------------------------ mat_fill_row_element */
template <typename SrcExp, typename ValExp, typename IndexExp, typename DType>
struct MatFillRowElementExp
    : public Exp<MatFillRowElementExp<SrcExp, ValExp, IndexExp, DType>, DType, type::kChainer> {
  const SrcExp &src_;
  const ValExp &val_;
  const IndexExp &index_;
  MatFillRowElementExp(const SrcExp &src, const ValExp &val, const IndexExp &index)
      : src_(src), val_(val), index_(index) {}
};
template <typename SrcExp, typename ValExp, typename IndexExp, typename SDType, typename VDType,
          typename IDType, int e1, int e2, int e3>
inline MatFillRowElementExp<SrcExp, ValExp, IndexExp, SDType> mat_fill_row_element(
    const Exp<SrcExp, SDType, e1> &src, const Exp<ValExp, VDType, e2> &val,
    const Exp<IndexExp, IDType, e3> &index) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim == 2 && ExpInfo<ValExp>::kDim == 1 &&
                ExpInfo<IndexExp>::kDim == 1>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return MatFillRowElementExp<SrcExp, ValExp, IndexExp, SDType>(src.self(), val.self(),
                                                                index.self());
}
template <typename SrcExp, typename ValExp, typename IndexExp, typename DType>
struct Plan<MatFillRowElementExp<SrcExp, ValExp, IndexExp, DType>, DType> {
 public:
  explicit Plan(const MatFillRowElementExp<SrcExp, ValExp, IndexExp, DType> &e)
      : src_(MakePlan(e.src_)), val_(MakePlan(e.val_)), index_(MakePlan(e.index_)) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    return static_cast<index_t>(index_.Eval(0, y)) == x ? static_cast<DType>(val_.Eval(0, y))
                                                         : static_cast<DType>(src_.Eval(y, x));
  }

 private:
  Plan<SrcExp, DType> src_;
  Plan<ValExp, DType> val_;
  Plan<IndexExp, DType> index_;
};
template <typename SrcExp, typename ValExp, typename IndexExp, typename DType>
inline Plan<MatFillRowElementExp<SrcExp, ValExp, IndexExp, DType>, DType> MakePlan(
    const MatFillRowElementExp<SrcExp, ValExp, IndexExp, DType> &exp) {
  return Plan<MatFillRowElementExp<SrcExp, ValExp, IndexExp, DType>, DType>(exp);
}
template <int dim, typename SrcExp, typename ValExp, typename IndexExp, typename DType>
struct ShapeCheck<dim, MatFillRowElementExp<SrcExp, ValExp, IndexExp, DType> > {
  inline static Shape<dim> Check(const MatFillRowElementExp<SrcExp, ValExp, IndexExp, DType> &t) {
    CHECK(dim == 2) << "MatFillRowElementExp only support 2 dimension output";
    Shape<2> sshape = ShapeCheck<2, SrcExp>::Check(t.src_);
    Shape<1> vshape = ShapeCheck<1, ValExp>::Check(t.val_);
    Shape<1> ishape = ShapeCheck<1, IndexExp>::Check(t.index_);
    CHECK((sshape[0] == ishape[0]) && (ishape[0] == vshape[0]))
        << "mat_fill_row_element index length, val length and number of rows in matrix";
    return sshape;
  }
};
template <typename SrcExp, typename ValExp, typename IndexExp, typename DType>
struct ExpInfo<MatFillRowElementExp<SrcExp, ValExp, IndexExp, DType> > {
  static const int kDim = 2;
  static const int kDevMask =
      ExpInfo<SrcExp>::kDevMask & ExpInfo<ValExp>::kDevMask & ExpInfo<IndexExp>::kDevMask;
};

/* ------------------------------------------------------------------ range */
/*! \brief start, start + step, ... (every value `repeat` times) up to but excluding stop */
template <typename DType>
struct RangeExp : public Exp<RangeExp<DType>, DType, type::kMapper> {
  const DType start_, stop_, step_;
  const int repeat_;
  RangeExp(DType start, DType stop, DType step, int repeat)
      : start_(start), stop_(stop), step_(step), repeat_(repeat) {}
};
template <typename DType>
inline RangeExp<DType> range(DType start, DType stop, DType step = 1, int repeat = 1) {
  return RangeExp<DType>(start, stop, step, repeat);
}
template <typename DType>
struct Plan<RangeExp<DType>, DType> {
 public:
  explicit Plan(const RangeExp<DType> &e) : start_(e.start_), step_(e.step_), repeat_(e.repeat_) {}
  MSHADOW_XINLINE DType Eval(index_t, index_t x) const {
    return start_ + static_cast<DType>(static_cast<int>(x) / repeat_) * step_;
  }

 private:
  const DType start_, step_;
  const int repeat_;
};
template <typename DType>
inline Plan<RangeExp<DType>, DType> MakePlan(const RangeExp<DType> &exp) {
  return Plan<RangeExp<DType>, DType>(exp);
}
/*! \brief element count of a range; integer types count by integer division, floating
 *  types by the ceiling of the quotient computed in double */
template <typename DType>
inline int RangeOutSize(DType start, DType stop, DType step, int repeat) {
  return repeat * ((stop - start - 1) / step + 1);
}
template <>
inline int RangeOutSize<float>(float start, float stop, float step, int repeat) {
  const double span = static_cast<double>(stop) - static_cast<double>(start);
  return repeat * static_cast<int>(ceil(span / static_cast<double>(step)));
}
template <>
inline int RangeOutSize<double>(double start, double stop, double step, int repeat) {
  return repeat * static_cast<int>(ceil((stop - start) / step));
}
template <int dim, typename DType>
struct ShapeCheck<dim, RangeExp<DType> > {
  inline static Shape<dim> Check(const RangeExp<DType> &t) {
    CHECK(dim == 1) << "RangeExp only support 1 dimension output, received " << dim;
    CHECK(t.step_ != 0) << "RangeExp does not support step=0, received " << t.step_;
    CHECK(t.repeat_ > 0) << "RangeExp only supports repeat > 0, received " << t.repeat_;
    if (t.step_ > 0) {
      CHECK(t.start_ < t.stop_) << "RangeExp does not support (start, stop, step) = "
                                << "(" << t.start_ << "," << t.stop_ << "," << t.step_ << ")";
    } else {
      CHECK(t.start_ > t.stop_) << "RangeExp does not support (start, stop, step)= "
                                << "(" << t.start_ << "," << t.stop_ << "," << t.step_ << ")";
    }
    return Shape1(RangeOutSize<DType>(t.start_, t.stop_, t.step_, t.repeat_));
  }
};
template <typename DType>
struct ExpInfo<RangeExp<DType> > {
  static const int kDim = 1;
  static const int kDevMask = 0xffff;
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_INDEXING_H_
