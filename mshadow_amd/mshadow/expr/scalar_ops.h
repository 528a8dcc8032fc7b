/*
 * Operators mixing an expression with a plain scalar: `0.5f * x`, `x + 1.0f`,
 * `F<op>(x, 2.0f)`, and `scale * sumall_except_dim<k>(x)`.
 *
 * The scalar side is taken as `const ScalarExp<T>&`, a non-deduced parameter, so a
 * bare literal converts implicitly (mshadow/expression.h:81). One set is stamped out
 * per scalar type: float, double, int32_t, int64_t, half_t - the same list as
 * mshadow/tensor.h:1066-1080 of the reference; overload shapes per
 * mshadow/expr_scalar-inl.h:20-162.
 */
#ifndef MSHADOW_EXPR_SCALAR_OPS_H_
#define MSHADOW_EXPR_SCALAR_OPS_H_

#include "../tensor.h"

namespace mshadow {
namespace expr {

#define MSHADOW_SCALAR_BINOP_(T, SYM, OP)                                                   \
  template <typename TA, int ta>                                                            \
  inline BinaryMapExp<OP, TA, ScalarExp<T>, T, (ta | type::kMapper)> operator SYM(          \
      const Exp<TA, T, ta> &lhs, const ScalarExp<T> &rhs) {                                 \
    return MakeExp<OP>(lhs, rhs);                                                           \
  }                                                                                         \
  template <typename TB, int tb>                                                            \
  inline BinaryMapExp<OP, ScalarExp<T>, TB, T, (tb | type::kMapper)> operator SYM(          \
      const ScalarExp<T> &lhs, const Exp<TB, T, tb> &rhs) {                                 \
    return MakeExp<OP>(lhs, rhs);                                                           \
  }                                                                                         \
  inline BinaryMapExp<OP, ScalarExp<T>, ScalarExp<T>, T, (1 | type::kMapper)> operator SYM( \
      const ScalarExp<T> &lhs, const ScalarExp<T> &rhs) {                                   \
    return MakeExp<OP>(lhs, rhs);                                                           \
  }

#define MSHADOW_SCALAR_OPS_(T)                                                              \
  /* scale folded into the dot / reduce node instead of a map */                            \
  template <typename TA, typename TB, bool ltrans, bool rtrans>                             \
  inline DotExp<TA, TB, ltrans, rtrans, T> operator*(                                       \
      const DotExp<TA, TB, ltrans, rtrans, T> &lhs, T rhs) {                                \
    return DotExp<TA, TB, ltrans, rtrans, T>(lhs.lhs_, lhs.rhs_, lhs.scale_ * rhs);         \
  }                                                                                         \
  template <typename TA, typename TB, bool ltrans, bool rtrans>                             \
  inline DotExp<TA, TB, ltrans, rtrans, T> operator*(                                       \
      T lhs, const DotExp<TA, TB, ltrans, rtrans, T> &rhs) {                                \
    return DotExp<TA, TB, ltrans, rtrans, T>(rhs.lhs_, rhs.rhs_, rhs.scale_ * lhs);         \
  }                                                                                         \
  template <typename E, typename DType, typename R, int d>                                  \
  inline ReduceTo1DExp<E, DType, R, d> operator*(const ReduceTo1DExp<E, DType, R, d> &e,    \
                                                 T scale) {                                 \
    return ReduceTo1DExp<E, DType, R, d>(e.src_, e.scale_ * scale);                         \
  }                                                                                         \
  template <typename E, typename DType, typename R, int d>                                  \
  inline ReduceTo1DExp<E, DType, R, d> operator*(T scale,                                   \
                                                 const ReduceTo1DExp<E, DType, R, d> &e) {  \
    return ReduceTo1DExp<E, DType, R, d>(e.src_, e.scale_ * scale);                         \
  }                                                                                         \
  /* F<OP>(expr, scalar) and friends */                                                     \
  template <typename OP, typename TA, int ta>                                               \
  inline BinaryMapExp<OP, TA, ScalarExp<T>, T, (ta | type::kMapper)> F(                     \
      const Exp<TA, T, ta> &lhs, const ScalarExp<T> &rhs) {                                 \
    return MakeExp<OP>(lhs, rhs);                                                           \
  }                                                                                         \
  template <typename OP, typename TB, int tb>                                               \
  inline BinaryMapExp<OP, ScalarExp<T>, TB, T, (tb | type::kMapper)> F(                     \
      const ScalarExp<T> &lhs, const Exp<TB, T, tb> &rhs) {                                 \
    return MakeExp<OP>(lhs, rhs);                                                           \
  }                                                                                         \
  template <typename OP>                                                                    \
  inline BinaryMapExp<OP, ScalarExp<T>, ScalarExp<T>, T, (1 | type::kMapper)> F(            \
      const ScalarExp<T> &lhs, const ScalarExp<T> &rhs) {                                   \
    return MakeExp<OP>(lhs, rhs);                                                           \
  }                                                                                         \
  MSHADOW_SCALAR_BINOP_(T, +, op::plus)                                                     \
  MSHADOW_SCALAR_BINOP_(T, -, op::minus)                                                    \
  MSHADOW_SCALAR_BINOP_(T, *, op::mul)                                                      \
  MSHADOW_SCALAR_BINOP_(T, /, op::div)

MSHADOW_SCALAR_OPS_(float)
MSHADOW_SCALAR_OPS_(double)
MSHADOW_SCALAR_OPS_(int32_t)
MSHADOW_SCALAR_OPS_(int64_t)
MSHADOW_SCALAR_OPS_(mshadow::half::half_t)

#undef MSHADOW_SCALAR_OPS_
#undef MSHADOW_SCALAR_BINOP_

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXPR_SCALAR_OPS_H_
