/*
 * Arithmetic on complex tensors stored interleaved: the last dimension holds
 * (real, imaginary) pairs, so a tensor of n complex numbers per row has 2 n columns.
 *   complex_mul_cc / _cr / _rc, complex_div_cc / _cr / _rc   complex (c) or real (r) operands
 *   conj, complex_exchange                                    complex -> complex
 *   complex_pad_imag                                          real -> complex (imaginary 0)
 *   complex_toreal, complex_abs_square, complex_sum_real_imag complex -> real
 * and ComplexF<calctype, OP>(...) for caller-defined operators with the same static
 * members as those of op::complex below.
 *
 * Semantics and operator interface restate mshadow/extension/complex.h:13-523 of the
 * reference: every output element re-reads the pair(s) it needs and evaluates its half of
 * the operator; products and sums are separate float operations in the order written there.
 * A complex-by-complex expression of pack-evaluable operands is evaluated two complex
 * numbers (one 128-bit pack) at a time.
 */
#ifndef MSHADOW_EXT_COMPLEX_H_
#define MSHADOW_EXT_COMPLEX_H_

#include <type_traits>

#include "../tensor.h"

namespace mshadow {
namespace op {
namespace complex {
enum BinaryCalculationType { kBinaryCC, kBinaryCR, kBinaryRC };
enum UnitaryCalculationType { kUnitaryC2R, kUnitaryC2C, kUnitaryR2C };

/* binary operators: halves of the result from the four parts of the operands */
struct mul {
  template <typename DType>
  MSHADOW_XINLINE static DType RealMap(DType a_real, DType a_imag, DType b_real, DType b_imag) {
    return a_real * b_real - a_imag * b_imag;
  }
  template <typename DType>
  MSHADOW_XINLINE static DType ImagMap(DType a_real, DType a_imag, DType b_real, DType b_imag) {
    return a_real * b_imag + b_real * a_imag;
  }
};
struct div {
  template <typename DType>
  MSHADOW_XINLINE static DType RealMap(DType a_real, DType a_imag, DType b_real, DType b_imag) {
    return (a_real * b_real + a_imag * b_imag) / (b_real * b_real + b_imag * b_imag);
  }
  template <typename DType>
  MSHADOW_XINLINE static DType ImagMap(DType a_real, DType a_imag, DType b_real, DType b_imag) {
    return (b_real * a_imag - a_real * b_imag) / (b_real * b_real + b_imag * b_imag);
  }
};

/* unitary operators: halves of the result from the source plan and the positions of the
   real and the imaginary part */
struct conjugate {
  template <typename TA, typename DType>
  MSHADOW_XINLINE static DType RealMap(const expr::Plan<TA, DType> &src, index_t real_i,
                                       index_t real_j, index_t, index_t) {
    return src.Eval(real_i, real_j);
  }
  template <typename TA, typename DType>
  MSHADOW_XINLINE static DType ImagMap(const expr::Plan<TA, DType> &src, index_t, index_t,
                                       index_t imag_i, index_t imag_j) {
    return -src.Eval(imag_i, imag_j);
  }
};
struct exchange {
  template <typename TA, typename DType>
  MSHADOW_XINLINE static DType RealMap(const expr::Plan<TA, DType> &src, index_t, index_t,
                                       index_t imag_i, index_t imag_j) {
    return src.Eval(imag_i, imag_j);
  }
  template <typename TA, typename DType>
  MSHADOW_XINLINE static DType ImagMap(const expr::Plan<TA, DType> &src, index_t real_i,
                                       index_t real_j, index_t, index_t) {
    return src.Eval(real_i, real_j);
  }
};
struct pad_imag {
  template <typename TA, typename DType>
  MSHADOW_XINLINE static DType RealMap(const expr::Plan<TA, DType> &src, index_t real_i,
                                       index_t real_j) {
    return src.Eval(real_i, real_j);
  }
  template <typename TA, typename DType>
  MSHADOW_XINLINE static DType ImagMap(const expr::Plan<TA, DType> &, index_t, index_t) {
    return 0;
  }
};
struct toreal {
  template <typename TA, typename DType>
  MSHADOW_XINLINE static DType RealMap(const expr::Plan<TA, DType> &src, index_t real_i,
                                       index_t real_j, index_t, index_t) {
    return src.Eval(real_i, real_j);
  }
};
struct abs_square {
  template <typename TA, typename DType>
  MSHADOW_XINLINE static DType RealMap(const expr::Plan<TA, DType> &src, index_t real_i,
                                       index_t real_j, index_t imag_i, index_t imag_j) {
    const DType re = src.Eval(real_i, real_j), im = src.Eval(imag_i, imag_j);
    return re * re + im * im;
  }
};
struct sum_real_imag {
  template <typename TA, typename DType>
  MSHADOW_XINLINE static DType RealMap(const expr::Plan<TA, DType> &src, index_t real_i,
                                       index_t real_j, index_t imag_i, index_t imag_j) {
    const DType re = src.Eval(real_i, real_j), im = src.Eval(imag_i, imag_j);
    return re + im;
  }
};
}  // namespace complex
}  // namespace op

namespace expr {

template <int calctype, typename OP, typename TA, typename TB, typename DType, int etype>
struct ComplexBinaryMapExp
    : public Exp<ComplexBinaryMapExp<calctype, OP, TA, TB, DType, etype>, DType, etype> {
  const TA &lhs_;
  const TB &rhs_;
  ComplexBinaryMapExp(const TA &lhs, const TB &rhs) : lhs_(lhs), rhs_(rhs) {}
};
template <int calctype, typename OP, typename TA, typename DType, int etype>
struct ComplexUnitaryExp
    : public Exp<ComplexUnitaryExp<calctype, OP, TA, DType, etype>, DType, etype> {
  const TA &src_;
  explicit ComplexUnitaryExp(const TA &src) : src_(src) {}
};

template <int calctype, typename OP, typename TA, typename TB, typename DType, int ta, int tb>
inline ComplexBinaryMapExp<calctype, OP, TA, TB, DType, (ta | tb | type::kMapper)> ComplexF(
    const Exp<TA, DType, ta> &lhs, const Exp<TB, DType, tb> &rhs) {
  return ComplexBinaryMapExp<calctype, OP, TA, TB, DType, (ta | tb | type::kMapper)>(lhs.self(),
                                                                                    rhs.self());
}
template <int calctype, typename OP, typename SrcExp, typename DType, int e1>
inline ComplexUnitaryExp<calctype, OP, SrcExp, DType, (e1 | type::kMapper)> ComplexF(
    const Exp<SrcExp, DType, e1> &src) {
  return ComplexUnitaryExp<calctype, OP, SrcExp, DType, (e1 | type::kMapper)>(src.self());
}

#define MSHADOW_COMPLEX_BINARY(NAME, CALC, OP)                                              \
  template <typename TA, typename TB, typename DType, int ta, int tb>                       \
  inline ComplexBinaryMapExp<op::complex::CALC, op::complex::OP, TA, TB, DType,             \
                             (ta | tb | type::kMapper)>                                     \
  NAME(const Exp<TA, DType, ta> &lhs, const Exp<TB, DType, tb> &rhs) {                      \
    return ComplexF<op::complex::CALC, op::complex::OP>(lhs, rhs);                          \
  }
MSHADOW_COMPLEX_BINARY(complex_mul_cc, kBinaryCC, mul)
MSHADOW_COMPLEX_BINARY(complex_mul_cr, kBinaryCR, mul)
MSHADOW_COMPLEX_BINARY(complex_mul_rc, kBinaryRC, mul)
MSHADOW_COMPLEX_BINARY(complex_div_cc, kBinaryCC, div)
MSHADOW_COMPLEX_BINARY(complex_div_cr, kBinaryCR, div)
MSHADOW_COMPLEX_BINARY(complex_div_rc, kBinaryRC, div)
#undef MSHADOW_COMPLEX_BINARY
#define MSHADOW_COMPLEX_UNITARY(NAME, CALC, OP)                                                  \
  template <typename SrcExp, typename DType, int e1>                                             \
  inline ComplexUnitaryExp<op::complex::CALC, op::complex::OP, SrcExp, DType,                    \
                           (e1 | type::kMapper)>                                                 \
  NAME(const Exp<SrcExp, DType, e1> &src) {                                                      \
    return ComplexF<op::complex::CALC, op::complex::OP>(src);                                    \
  }
MSHADOW_COMPLEX_UNITARY(conj, kUnitaryC2C, conjugate)
MSHADOW_COMPLEX_UNITARY(complex_exchange, kUnitaryC2C, exchange)
MSHADOW_COMPLEX_UNITARY(complex_pad_imag, kUnitaryR2C, pad_imag)
MSHADOW_COMPLEX_UNITARY(complex_toreal, kUnitaryC2R, toreal)
MSHADOW_COMPLEX_UNITARY(complex_abs_square, kUnitaryC2R, abs_square)
MSHADOW_COMPLEX_UNITARY(complex_sum_real_imag, kUnitaryC2R, sum_real_imag)
#undef MSHADOW_COMPLEX_UNITARY

/* ---- shapes: a complex operand has an even last dimension, a real one half of it ---- */
template <int dim, int calctype, typename OP, typename TA, typename TB, typename DType, int etype>
struct ShapeCheck<dim, ComplexBinaryMapExp<calctype, OP, TA, TB, DType, etype> > {
  inline static Shape<dim> Check(
      const ComplexBinaryMapExp<calctype, OP, TA, TB, DType, etype> &t) {
    Shape<dim> lhs = ShapeCheck<dim, TA>::Check(t.lhs_);
    Shape<dim> rhs = ShapeCheck<dim, TB>::Check(t.rhs_);
    if (lhs[0] == 0) return rhs;
    if (rhs[0] == 0) return lhs;
    if (calctype == op::complex::kBinaryCC) {
      CHECK_EQ(lhs, rhs) << "ComplexBinaryMapExp (CC): Shapes of operands are not the same.";
      CHECK_EQ(lhs[dim - 1] % 2, 0)
          << "ComplexBinaryMapExp (CC): Shape of the last dimension is not even. "
             "We must have real part + imaginary part.";
      return lhs;
    }
    const char *kind = calctype == op::complex::kBinaryCR ? "CR" : "RC";
    CHECK(calctype == op::complex::kBinaryCR || calctype == op::complex::kBinaryRC)
        << "ComplexBinaryMapExp: Unexpected Calculation Type!";
    for (int i = 0; i < dim - 1; ++i) {
      CHECK_EQ(lhs[i], rhs[i]) << "ComplexBinaryMapExp (" << kind
                               << "): Shapes of operands are not the same.";
    }
    const Shape<dim> &wide = calctype == op::complex::kBinaryCR ? lhs : rhs;
    const Shape<dim> &narrow = calctype == op::complex::kBinaryCR ? rhs : lhs;
    CHECK_EQ(wide[dim - 1], narrow[dim - 1] * 2)
        << "ComplexBinaryMapExp (" << kind << "): Shapes of operands do not match.";
    return wide;
  }
};
template <int dim, int calctype, typename OP, typename TA, typename DType, int etype>
struct ShapeCheck<dim, ComplexUnitaryExp<calctype, OP, TA, DType, etype> > {
  inline static Shape<dim> Check(const ComplexUnitaryExp<calctype, OP, TA, DType, etype> &t) {
    Shape<dim> s = ShapeCheck<dim, TA>::Check(t.src_);
    /* checked for real sources too, as the reference does */
    CHECK_EQ(s[dim - 1] % 2, 0) << "ComplexUnitaryExp: Shape of the last dimension is not even. "
                                   "We must have real + imaginary.";
    if (calctype == op::complex::kUnitaryC2R) s[dim - 1] /= 2;
    if (calctype == op::complex::kUnitaryR2C) s[dim - 1] *= 2;
    return s;
  }
};

/* ---- plans ---- */
namespace complex_detail {
/*! \brief the (real, imaginary) parts an operand contributes to the complex number that
 *  starts at column base_x of the result: its own pair, or its real value and a zero */
template <bool kIsComplex>
struct Parts {
  template <typename P, typename DType>
  MSHADOW_XINLINE static void Get(const P &plan, index_t y, index_t base_x, DType *re, DType *im) {
    *re = plan.Eval(y, base_x);
    *im = plan.Eval(y, base_x + 1);
  }
};
template <>
struct Parts<false> {
  template <typename P, typename DType>
  MSHADOW_XINLINE static void Get(const P &plan, index_t y, index_t base_x, DType *re, DType *im) {
    *re = plan.Eval(y, base_x / 2);
    *im = static_cast<DType>(0);
  }
};
}  // namespace complex_detail

template <int calctype, typename OP, typename TA, typename TB, int etype, typename DType>
class Plan<ComplexBinaryMapExp<calctype, OP, TA, TB, DType, etype>, DType> {
 public:
  Plan(const Plan<TA, DType> &lhs, const Plan<TB, DType> &rhs) : lhs_(lhs), rhs_(rhs) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    const index_t base_x = (x / 2) * 2;
    DType ar, ai, br, bi;
    complex_detail::Parts<calctype != op::complex::kBinaryRC>::Get(lhs_, y, base_x, &ar, &ai);
    complex_detail::Parts<calctype != op::complex::kBinaryCR>::Get(rhs_, y, base_x, &br, &bi);
    return x % 2 == 0 ? OP::RealMap(ar, ai, br, bi) : OP::ImagMap(ar, ai, br, bi);
  }
  /* complex by complex: a pack holds whole pairs of both operands */
  static const bool kPackable = calctype == op::complex::kBinaryCC &&
                                plan_detail::Packable<Plan<TA, DType> >::value &&
                                plan_detail::Packable<Plan<TB, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    const Pack<DType, N> a = lhs_.template EvalPack<N, STREAM>(y, x);
    const Pack<DType, N> b = rhs_.template EvalPack<N, STREAM>(y, x);
    Pack<DType, N> r;
#pragma unroll
    for (int k = 0; k + 1 < N; k += 2) {
      r.v[k] = OP::RealMap(a.v[k], a.v[k + 1], b.v[k], b.v[k + 1]);
      r.v[k + 1] = OP::ImagMap(a.v[k], a.v[k + 1], b.v[k], b.v[k + 1]);
    }
    return r;
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    return n % 2 == 0 && lhs_.PackReady(n, cols, flat) && rhs_.PackReady(n, cols, flat);
  }

 private:
  Plan<TA, DType> lhs_;
  Plan<TB, DType> rhs_;
};

template <int calctype, typename OP, typename TA, int etype, typename DType>
class Plan<ComplexUnitaryExp<calctype, OP, TA, DType, etype>, DType> {
 public:
  explicit Plan(const Plan<TA, DType> &src) : src_(src) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const { return Half<calctype>(y, x); }

 private:
  /* complex -> complex: the pair sits where the result's pair sits */
  template <int kCalc>
  MSHADOW_XINLINE typename std::enable_if<kCalc == op::complex::kUnitaryC2C, DType>::type Half(
      index_t y, index_t x) const {
    const index_t base_x = (x / 2) * 2;
    return x % 2 == 0 ? OP::RealMap(src_, y, base_x, y, base_x + 1)
                      : OP::ImagMap(src_, y, base_x, y, base_x + 1);
  }
  /* real -> complex: column x / 2 of the source feeds both halves */
  template <int kCalc>
  MSHADOW_XINLINE typename std::enable_if<kCalc == op::complex::kUnitaryR2C, DType>::type Half(
      index_t y, index_t x) const {
    return x % 2 == 0 ? OP::RealMap(src_, y, x / 2) : OP::ImagMap(src_, y, x / 2);
  }
  /* complex -> real: the pair at columns 2 x, 2 x + 1 */
  template <int kCalc>
  MSHADOW_XINLINE typename std::enable_if<kCalc == op::complex::kUnitaryC2R, DType>::type Half(
      index_t y, index_t x) const {
    return OP::RealMap(src_, y, x * 2, y, x * 2 + 1);
  }
  Plan<TA, DType> src_;
};

template <int calctype, typename OP, typename TA, typename TB, typename DType, int etype>
inline Plan<ComplexBinaryMapExp<calctype, OP, TA, TB, DType, etype>, DType> MakePlan(
    const ComplexBinaryMapExp<calctype, OP, TA, TB, DType, etype> &e) {
  return Plan<ComplexBinaryMapExp<calctype, OP, TA, TB, DType, etype>, DType>(MakePlan(e.lhs_),
                                                                              MakePlan(e.rhs_));
}
template <int calctype, typename OP, typename TA, typename DType, int etype>
inline Plan<ComplexUnitaryExp<calctype, OP, TA, DType, etype>, DType> MakePlan(
    const ComplexUnitaryExp<calctype, OP, TA, DType, etype> &e) {
  return Plan<ComplexUnitaryExp<calctype, OP, TA, DType, etype>, DType>(MakePlan(e.src_));
}

template <int calctype, typename OP, typename TA, typename TB, typename DType, int etype>
struct ExpInfo<ComplexBinaryMapExp<calctype, OP, TA, TB, DType, etype> > {
  static const int kDimLhs = ExpInfo<TA>::kDim;
  static const int kDimRhs = ExpInfo<TB>::kDim;
  static const int kDim =
      (kDimLhs < 0 || kDimRhs < 0) ? -1
      : (kDimLhs == 0)             ? kDimRhs
      : (kDimRhs == 0 || kDimLhs == kDimRhs) ? kDimLhs : -1;
  static const int kDevMask = ExpInfo<TA>::kDevMask & ExpInfo<TB>::kDevMask;
};
template <int calctype, typename OP, typename TA, typename DType, int etype>
struct ExpInfo<ComplexUnitaryExp<calctype, OP, TA, DType, etype> > {
  static const int kDim = ExpInfo<TA>::kDim;
  static const int kDevMask = ExpInfo<TA>::kDevMask;
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_COMPLEX_H_
