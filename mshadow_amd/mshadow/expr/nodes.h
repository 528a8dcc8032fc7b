/*
 * Expression-tree node types of the mshadow API.
 *
 * `dst = a * b + F<op>(c)` builds, at compile time, a tree of the small structs below;
 * nothing is computed until the assignment hands the tree to ExpEngine. The node
 * names, template parameter orders and the operator set follow
 * mshadow/expression.h:60-413 of the reference so that caller code compiles
 * unchanged. Nodes hold their children by const reference: a tree is only valid
 * inside the full expression that created it.
 */
#ifndef MSHADOW_EXPR_NODES_H_
#define MSHADOW_EXPR_NODES_H_

#include "../base.h"

namespace mshadow {
namespace expr {

/*! \brief category of an expression node, a bit set combined with | when nodes nest */
namespace type {
const int kRValue = 0;   //!< storage that can be assigned to
const int kMapper = 1;   //!< element-to-same-element map
const int kChainer = 3;  //!< element-to-other-element map (pool, pad, ...)
const int kComplex = 7;  //!< needs its own engine (dot, reduce-to-1D)
}  // namespace type

template <typename Saver, typename RValue, typename DType>
struct ExpEngine;

/*! \brief CRTP root of every expression */
template <typename SubType, typename DType, int exp_type>
struct Exp {
  inline const SubType &self(void) const { return *static_cast<const SubType *>(this); }
  inline SubType *ptrself(void) { return static_cast<SubType *>(this); }
};

/*! \brief a constant broadcast to every element */
template <typename DType>
struct ScalarExp : public Exp<ScalarExp<DType>, DType, type::kMapper> {
  DType scalar_;
  ScalarExp(DType scalar) : scalar_(scalar) {}  // NOLINT(*) implicit on purpose
};
template <typename DType>
inline ScalarExp<DType> scalar(DType s) {
  return ScalarExp<DType>(s);
}

/*! \brief element type conversion, DstDType(value) */
template <typename DstDType, typename SrcDType, typename EType, int etype>
struct TypecastExp : public Exp<TypecastExp<DstDType, SrcDType, EType, etype>, DstDType, etype> {
  const EType &exp;
  explicit TypecastExp(const EType &e) : exp(e) {}
};
template <typename DstDType, typename SrcDType, typename EType, int etype>
inline TypecastExp<DstDType, SrcDType, EType, (etype | type::kMapper)> tcast(
    const Exp<EType, SrcDType, etype> &exp) {
  return TypecastExp<DstDType, SrcDType, EType, (etype | type::kMapper)>(exp.self());
}

/*! \brief transposed view of a 2-D expression */
template <typename EType, typename DType>
struct TransposeExp : public Exp<TransposeExp<EType, DType>, DType, type::kChainer> {
  const EType &exp;
  explicit TransposeExp(const EType &e) : exp(e) {}
  inline const EType &T(void) const { return exp; }
};

/*! \brief anything that can stand on the left of an assignment */
template <typename Container, typename DType>
class RValueExp : public Exp<Container, DType, type::kRValue> {
 public:
  inline const TransposeExp<Container, DType> T(void) const {
    return TransposeExp<Container, DType>(this->self());
  }
#define MSHADOW_RVALUE_ASSIGN(NAME, SAVER)                                          \
  inline Container &NAME(DType s) {                                                 \
    ExpEngine<SAVER, Container, DType>::Eval(this->ptrself(), scalar<DType>(s));    \
    return *(this->ptrself());                                                      \
  }                                                                                 \
  template <typename E, int etype>                                                  \
  inline Container &NAME(const Exp<E, DType, etype> &exp) {                         \
    ExpEngine<SAVER, Container, DType>::Eval(this->ptrself(), exp.self());          \
    return *(this->ptrself());                                                      \
  }
  MSHADOW_RVALUE_ASSIGN(operator+=, sv::plusto)
  MSHADOW_RVALUE_ASSIGN(operator-=, sv::minusto)
  MSHADOW_RVALUE_ASSIGN(operator*=, sv::multo)
  MSHADOW_RVALUE_ASSIGN(operator/=, sv::divto)
  MSHADOW_RVALUE_ASSIGN(__assign, sv::saveto)
#undef MSHADOW_RVALUE_ASSIGN
  inline Container &__assign(const Exp<Container, DType, type::kRValue> &exp);
};

/*! \brief matrix product node; its engine (BLAS) is not part of this backend */
template <typename TA, typename TB, bool ltrans, bool rtrans, typename DType>
struct DotExp : public Exp<DotExp<TA, TB, ltrans, rtrans, DType>, DType, type::kComplex> {
  const TA &lhs_;
  const TB &rhs_;
  DType scale_;
  explicit DotExp(const TA &lhs, const TB &rhs, DType scale) : lhs_(lhs), rhs_(rhs), scale_(scale) {}
};
template <typename TA, typename TB, typename DType>
inline DotExp<TA, TB, false, false, DType> dot(const RValueExp<TA, DType> &lhs,
                                               const RValueExp<TB, DType> &rhs) {
  return DotExp<TA, TB, false, false, DType>(lhs.self(), rhs.self(), DType(1.0f));
}
template <typename TA, typename TB, typename DType>
inline DotExp<TA, TB, true, false, DType> dot(const TransposeExp<TA, DType> &lhs,
                                              const RValueExp<TB, DType> &rhs) {
  return DotExp<TA, TB, true, false, DType>(lhs.exp, rhs.self(), DType(1.0f));
}
template <typename TA, typename TB, typename DType>
inline DotExp<TA, TB, false, true, DType> dot(const RValueExp<TA, DType> &lhs,
                                              const TransposeExp<TB, DType> &rhs) {
  return DotExp<TA, TB, false, true, DType>(lhs.self(), rhs.exp, DType(1.0f));
}
template <typename TA, typename TB, typename DType>
inline DotExp<TA, TB, true, true, DType> dot(const TransposeExp<TA, DType> &lhs,
                                             const TransposeExp<TB, DType> &rhs) {
  return DotExp<TA, TB, true, true, DType>(lhs.exp, rhs.exp, DType(1.0f));
}
template <bool transpose_left, bool transpose_right, typename TA, typename TB, typename DType>
inline DotExp<TA, TB, transpose_left, transpose_right, DType> batch_dot(
    const RValueExp<TA, DType> &lhs, const RValueExp<TB, DType> &rhs) {
  return DotExp<TA, TB, transpose_left, transpose_right, DType>(lhs.self(), rhs.self(),
                                                                DType(1.0f));
}

/*! \brief OP::Map(a, b, c) per element */
template <typename OP, typename TA, typename TB, typename TC, typename DType, int etype>
struct TernaryMapExp : public Exp<TernaryMapExp<OP, TA, TB, TC, DType, etype>, DType, etype> {
  const TA &item1_;
  const TB &item2_;
  const TC &item3_;
  explicit TernaryMapExp(const TA &item1, const TB &item2, const TC &item3)
      : item1_(item1), item2_(item2), item3_(item3) {}
};
/*! \brief OP::Map(a, b) per element */
template <typename OP, typename TA, typename TB, typename DType, int etype>
struct BinaryMapExp : public Exp<BinaryMapExp<OP, TA, TB, DType, etype>, DType, etype> {
  const TA &lhs_;
  const TB &rhs_;
  explicit BinaryMapExp(const TA &lhs, const TB &rhs) : lhs_(lhs), rhs_(rhs) {}
};
/*! \brief OP::Map(a) per element */
template <typename OP, typename TA, typename DType, int etype>
struct UnaryMapExp : public Exp<UnaryMapExp<OP, TA, DType, etype>, DType, etype> {
  const TA &src_;
  explicit UnaryMapExp(const TA &src) : src_(src) {}
};

template <typename OP, typename TA, typename TB, typename TC, typename DType, int ta, int tb, int tc>
inline TernaryMapExp<OP, TA, TB, TC, DType, (ta | tb | tc | type::kMapper)> MakeExp(
    const Exp<TA, DType, ta> &item1, const Exp<TB, DType, tb> &item2,
    const Exp<TC, DType, tc> &item3) {
  return TernaryMapExp<OP, TA, TB, TC, DType, (ta | tb | tc | type::kMapper)>(
      item1.self(), item2.self(), item3.self());
}
template <typename OP, typename TA, typename TB, typename DType, int ta, int tb>
inline BinaryMapExp<OP, TA, TB, DType, (ta | tb | type::kMapper)> MakeExp(
    const Exp<TA, DType, ta> &lhs, const Exp<TB, DType, tb> &rhs) {
  return BinaryMapExp<OP, TA, TB, DType, (ta | tb | type::kMapper)>(lhs.self(), rhs.self());
}
template <typename OP, typename TA, typename DType, int ta>
inline UnaryMapExp<OP, TA, DType, (ta | type::kMapper)> MakeExp(const Exp<TA, DType, ta> &src) {
  return UnaryMapExp<OP, TA, DType, (ta | type::kMapper)>(src.self());
}

/*! \brief F<OP>(...) : apply a caller-supplied functor elementwise (1, 2 or 3 operands) */
template <typename OP, typename TA, typename TB, typename TC, typename DType, int ta, int tb, int tc>
inline TernaryMapExp<OP, TA, TB, TC, DType, (ta | tb | tc | type::kMapper)> F(
    const Exp<TA, DType, ta> &item1, const Exp<TB, DType, tb> &item2,
    const Exp<TC, DType, tc> &item3) {
  return MakeExp<OP>(item1, item2, item3);
}
template <typename OP, typename TA, typename TB, typename DType, int ta, int tb>
inline BinaryMapExp<OP, TA, TB, DType, (ta | tb | type::kMapper)> F(const Exp<TA, DType, ta> &lhs,
                                                                    const Exp<TB, DType, tb> &rhs) {
  return MakeExp<OP>(lhs, rhs);
}
template <typename OP, typename TA, typename DType, int ta>
inline UnaryMapExp<OP, TA, DType, (ta | type::kMapper)> F(const Exp<TA, DType, ta> &src) {
  return MakeExp<OP>(src);
}

#define MSHADOW_BINARY_OPERATOR(SYM, OP)                                                  \
  template <typename TA, typename TB, typename DType, int ta, int tb>                     \
  inline BinaryMapExp<OP, TA, TB, DType, (ta | tb | type::kMapper)> operator SYM(         \
      const Exp<TA, DType, ta> &lhs, const Exp<TB, DType, tb> &rhs) {                     \
    return MakeExp<OP>(lhs, rhs);                                                         \
  }
MSHADOW_BINARY_OPERATOR(+, op::plus)
MSHADOW_BINARY_OPERATOR(-, op::minus)
MSHADOW_BINARY_OPERATOR(*, op::mul)
MSHADOW_BINARY_OPERATOR(/, op::div)
#undef MSHADOW_BINARY_OPERATOR

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXPR_NODES_H_
