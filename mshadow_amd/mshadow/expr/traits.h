/*
 * Compile-time and run-time checks on expression trees:
 *   ExpInfo<E>     dimension and device mask of a tree (static)
 *   TypeCheck      can E be assigned to / reduced into a dim-d tensor on Device (static)
 *   ShapeCheck     the run-time shape of a tree, CHECK-failing on mismatch
 *   StreamInfo     which stream an assignment runs on (taken from the destination)
 * Contract: mshadow/expr_engine-inl.h:234-426 of the reference. A scalar has
 * dimension 0 and an all-zero shape, which every binary check skips.
 */
#ifndef MSHADOW_EXPR_TRAITS_H_
#define MSHADOW_EXPR_TRAITS_H_

#include <algorithm>
#include <utility>

#include "./plan.h"

namespace mshadow {
namespace expr {

template <typename E>
struct ExpInfo {
  static const int kDim = -1;
  static const int kDevMask = 0;
};
template <typename DType>
struct ExpInfo<ScalarExp<DType> > {
  static const int kDim = 0;
  static const int kDevMask = 0xffff;
};
template <typename E, typename DType>
struct ExpInfo<TransposeExp<E, DType> > {
  static const int kDim = ExpInfo<E>::kDim;
  static const int kDevMask = ExpInfo<E>::kDevMask;
};
template <typename DstDType, typename SrcDType, typename EType, int etype>
struct ExpInfo<TypecastExp<DstDType, SrcDType, EType, etype> > {
  static const int kDim = ExpInfo<EType>::kDim;
  static const int kDevMask = ExpInfo<EType>::kDevMask;
};
template <typename Device, int dim, typename DType>
struct ExpInfo<Tensor<Device, dim, DType> > {
  static const int kDim = dim;
  static const int kDevMask = Device::kDevMask;
};
template <typename T, typename SrcExp, int dim, typename DType>
struct ExpInfo<MakeTensorExp<T, SrcExp, dim, DType> > {
  static const int kDimSrc = ExpInfo<SrcExp>::kDim;
  static const int kDim = kDimSrc >= 0 ? dim : -1;
  static const int kDevMask = ExpInfo<SrcExp>::kDevMask;
};
template <typename OP, typename TA, typename DType, int etype>
struct ExpInfo<UnaryMapExp<OP, TA, DType, etype> > {
  static const int kDim = ExpInfo<TA>::kDim;
  static const int kDevMask = ExpInfo<TA>::kDevMask;
};
template <typename OP, typename TA, typename TB, typename DType, int etype>
struct ExpInfo<BinaryMapExp<OP, TA, TB, DType, etype> > {
  static const int kDimLhs = ExpInfo<TA>::kDim;
  static const int kDimRhs = ExpInfo<TB>::kDim;
  /* scalar (0) adopts the other side; otherwise both sides must agree */
  static const int kDim =
      (kDimLhs < 0 || kDimRhs < 0) ? -1
      : (kDimLhs == 0)             ? kDimRhs
      : (kDimRhs == 0 || kDimLhs == kDimRhs) ? kDimLhs : -1;
  static const int kDevMask = ExpInfo<TA>::kDevMask & ExpInfo<TB>::kDevMask;
};
template <typename OP, typename TA, typename TB, typename TC, typename DType, int etype>
struct ExpInfo<TernaryMapExp<OP, TA, TB, TC, DType, etype> > {
  static const int kDimItem1 = ExpInfo<TA>::kDim;
  static const int kDimItem2 = ExpInfo<TB>::kDim;
  static const int kDimItem3 = ExpInfo<TC>::kDim;
  static const int kDim = kDimItem1;
  static const int kDevMask =
      ExpInfo<TA>::kDevMask & ExpInfo<TB>::kDevMask & ExpInfo<TC>::kDevMask;
};

template <typename Device, int dim, typename DType, typename E>
struct TypeCheck {
  static const int kExpDim = ExpInfo<E>::kDim;
  static const bool kDevPass = (ExpInfo<E>::kDevMask & Device::kDevMask) != 0;
  /*! \brief E can be mapped elementwise onto a dim-d tensor */
  static const bool kMapPass = (kExpDim == 0 || kExpDim == dim) && kDevPass;
  /*! \brief E has more dimensions than the target, so it can be reduced into it */
  static const bool kRedPass = (kExpDim > dim) && kDevPass;
};
/*! \brief the member functions only exist for <true>: a failed check is a compile error
 *  whose text names the problem */
template <bool kPass>
struct TypeCheckPass;
template <>
struct TypeCheckPass<false> {};
template <>
struct TypeCheckPass<true> {
  inline static void Error_All_Tensor_in_Exp_Must_Have_Same_Type(void) {}
  inline static void Error_TypeCheck_Not_Pass_For_Reduce_Exp(void) {}
  inline static void Error_Expression_Does_Not_Meet_Dimension_Req(void) {}
};

template <typename Device, typename E>
struct StreamInfo {
  inline static Stream<Device> *Get(const E &t);
};
template <int dim, typename Device, typename DType>
struct StreamInfo<Device, Tensor<Device, dim, DType> > {
  inline static Stream<Device> *Get(const Tensor<Device, dim, DType> &t) { return t.stream_; }
};

template <int dim, typename E>
struct ShapeCheck {
  inline static Shape<dim> Check(const E &t);
};
template <int dim, typename DType>
struct ShapeCheck<dim, ScalarExp<DType> > {
  inline static Shape<dim> Check(const ScalarExp<DType> &exp) {
    Shape<dim> shape;
    for (int i = 0; i < dim; ++i) shape[i] = 0;
    return shape;
  }
};
template <int dim, typename DstDType, typename SrcDType, typename EType, int etype>
struct ShapeCheck<dim, TypecastExp<DstDType, SrcDType, EType, etype> > {
  inline static Shape<dim> Check(const TypecastExp<DstDType, SrcDType, EType, etype> &exp) {
    return ShapeCheck<dim, EType>::Check(exp.exp);
  }
};
template <int dim, typename E, typename DType>
struct ShapeCheck<dim, TransposeExp<E, DType> > {
  inline static Shape<dim> Check(const TransposeExp<E, DType> &e) {
    Shape<dim> s = ShapeCheck<dim, E>::Check(e.exp);
    std::swap(s[0], s[1]);
    return s;
  }
};
template <int dim, typename Device, typename DType>
struct ShapeCheck<dim, Tensor<Device, dim, DType> > {
  inline static Shape<dim> Check(const Tensor<Device, dim, DType> &t) { return t.shape_; }
};
template <int dim, typename SrcExp, typename T, typename DType>
struct ShapeCheck<dim, MakeTensorExp<T, SrcExp, dim, DType> > {
  inline static Shape<dim> Check(const MakeTensorExp<T, SrcExp, dim, DType> &t) {
    return t.shape_;
  }
};
template <int dim, typename OP, typename TA, typename DType, int etype>
struct ShapeCheck<dim, UnaryMapExp<OP, TA, DType, etype> > {
  inline static Shape<dim> Check(const UnaryMapExp<OP, TA, DType, etype> &t) {
    return ShapeCheck<dim, TA>::Check(t.src_);
  }
};
template <int dim, typename OP, typename TA, typename TB, typename DType, int etype>
struct ShapeCheck<dim, BinaryMapExp<OP, TA, TB, DType, etype> > {
  inline static Shape<dim> Check(const BinaryMapExp<OP, TA, TB, DType, etype> &t) {
    Shape<dim> lhs = ShapeCheck<dim, TA>::Check(t.lhs_);
    Shape<dim> rhs = ShapeCheck<dim, TB>::Check(t.rhs_);
    if (lhs[0] == 0) return rhs;
    if (rhs[0] == 0) return lhs;
    CHECK_EQ(lhs, rhs) << "BinaryMapExp: Shapes of operands are not the same, "
                       << "Shape1=" << lhs << ", Shape2=" << rhs;
    return lhs;
  }
};
template <int dim, typename OP, typename TA, typename TB, typename TC, typename DType, int etype>
struct ShapeCheck<dim, TernaryMapExp<OP, TA, TB, TC, DType, etype> > {
  inline static Shape<dim> Check(const TernaryMapExp<OP, TA, TB, TC, DType, etype> &t) {
    Shape<dim> s1 = ShapeCheck<dim, TA>::Check(t.item1_);
    Shape<dim> s2 = ShapeCheck<dim, TB>::Check(t.item2_);
    Shape<dim> s3 = ShapeCheck<dim, TC>::Check(t.item3_);
    CHECK((s1 == s2) && (s2 == s3))
        << "TernaryMapExp: Shapes of operands are not the same, "
        << "Shape1=" << s1 << ", Shape2=" << s2 << ", Shape3=" << s3;
    return s1;
  }
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXPR_TRAITS_H_
