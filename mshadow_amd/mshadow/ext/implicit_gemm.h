/*
 * implicit_dot(lhs, rhs): a matrix product evaluated element by element inside the
 * enclosing assignment, out(y, x) = sum over i of lhs(y, i) * rhs(i, x), for operands that
 * are themselves expressions and too small to be worth a BLAS call.
 *
 * Restates mshadow/extension/implicit_gemm.h:15-127 of the reference, whose evaluation order
 * is that of its 4-wide float packets (mshadow/packet/sse-inl.h:20-58): four running sums,
 * sum j taking the products of positions i with i % 4 == j of the largest multiple-of-4
 * prefix (each product rounded, then added); the four are combined as (s0 + s2) + (s1 + s3);
 * the remaining positions are then added one by one. Element types other than float use
 * the packet width of their size on a 16-byte vector in the reference; here every type
 * follows the rule with 16 / sizeof(DType) running sums (two for double, combined s0 + s1).
 */
#ifndef MSHADOW_EXT_IMPLICIT_GEMM_H_
#define MSHADOW_EXT_IMPLICIT_GEMM_H_

#include "../tensor.h"

namespace mshadow {
namespace expr {

template <typename LhsExp, typename RhsExp, typename DType>
struct ImplicitGEMMExp
    : public Exp<ImplicitGEMMExp<LhsExp, RhsExp, DType>, DType, type::kChainer> {
  const LhsExp &lhs_;
  const RhsExp &rhs_;
  index_t prod_size_;  //!< length of the contracted dimension
  Shape<2> shape_;
  ImplicitGEMMExp(const LhsExp &lhs, const RhsExp &rhs) : lhs_(lhs), rhs_(rhs) {
    Shape<2> slhs = ShapeCheck<2, LhsExp>::Check(lhs_);
    Shape<2> srhs = ShapeCheck<2, RhsExp>::Check(rhs_);
    shape_ = Shape2(slhs[0], srhs[1]);
    prod_size_ = slhs[1];
  }
};
template <typename LhsExp, typename RhsExp, typename DType, int e1, int e2>
inline ImplicitGEMMExp<LhsExp, RhsExp, DType> implicit_dot(const Exp<LhsExp, DType, e1> &lhs,
                                                           const Exp<RhsExp, DType, e2> &rhs) {
  TypeCheckPass<ExpInfo<LhsExp>::kDim == 2 && ExpInfo<RhsExp>::kDim == 2>::
      Error_Expression_Does_Not_Meet_Dimension_Req();
  return ImplicitGEMMExp<LhsExp, RhsExp, DType>(lhs.self(), rhs.self());
}

template <typename LhsExp, typename RhsExp, typename DType>
struct Plan<ImplicitGEMMExp<LhsExp, RhsExp, DType>, DType> {
 public:
  static const int kLanes = sizeof(DType) <= 16 ? 16 / sizeof(DType) : 1;
  explicit Plan(const ImplicitGEMMExp<LhsExp, RhsExp, DType> &e)
      : lhs_(MakePlan(e.lhs_)), rhs_(MakePlan(e.rhs_)), prod_size_(e.prod_size_),
        whole_(e.prod_size_ / kLanes * kLanes) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    DType part[kLanes];
#pragma unroll
    for (int j = 0; j < kLanes; ++j) part[j] = DType(0);
    for (index_t i = 0; i < whole_; i += kLanes) {
#pragma unroll
      for (int j = 0; j < kLanes; ++j) part[j] = part[j] + lhs_.Eval(y, i + j) * rhs_.Eval(i + j, x);
    }
    /* halves folded onto each other until one value is left: (s0 + s2) + (s1 + s3) */
#pragma unroll
    for (int width = kLanes / 2; width >= 1; width /= 2) {
#pragma unroll
      for (int j = 0; j < width; ++j) part[j] = part[j] + part[j + width];
    }
    DType res = part[0];
    for (index_t i = whole_; i < prod_size_; ++i) res += lhs_.Eval(y, i) * rhs_.Eval(i, x);
    return res;
  }

 private:
  Plan<LhsExp, DType> lhs_;
  Plan<RhsExp, DType> rhs_;
  const index_t prod_size_, whole_;
};
template <typename LhsExp, typename RhsExp, typename DType>
inline Plan<ImplicitGEMMExp<LhsExp, RhsExp, DType>, DType> MakePlan(
    const ImplicitGEMMExp<LhsExp, RhsExp, DType> &exp) {
  return Plan<ImplicitGEMMExp<LhsExp, RhsExp, DType>, DType>(exp);
}
template <int dim, typename LhsExp, typename RhsExp, typename DType>
struct ShapeCheck<dim, ImplicitGEMMExp<LhsExp, RhsExp, DType> > {
  inline static Shape<dim> Check(const ImplicitGEMMExp<LhsExp, RhsExp, DType> &t) {
    CHECK(dim == 2) << "ImplicitGEMMExp only support 2 dimension";
    Shape<dim> lhs = ShapeCheck<dim, LhsExp>::Check(t.lhs_);
    Shape<dim> rhs = ShapeCheck<dim, RhsExp>::Check(t.rhs_);
    CHECK_EQ(lhs[1], rhs[0]) << "implicit_dot The matrix shape do  not match";
    return t.shape_;
  }
};
template <typename LhsExp, typename RhsExp, typename DType>
struct ExpInfo<ImplicitGEMMExp<LhsExp, RhsExp, DType> > {
  static const int kDim = 2;
  static const int kDevMask = ExpInfo<LhsExp>::kDevMask & ExpInfo<RhsExp>::kDevMask;
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_IMPLICIT_GEMM_H_
