/*
 * ExpEngine: where `dst <saver>= expression` lands. Mapper, chainer and rvalue
 * trees go to MapExp on the destination's device; complex trees (reduce-to-1D, dot)
 * go to an ExpComplexEngine specialisation. Contract:
 * mshadow/expr_engine-inl.h:436-479 of the reference. The specialisation for DotExp
 * is in dot_engine.h, the one for reduce-to-1D in ext/reduceto1d.h.
 */
#ifndef MSHADOW_EXPR_ENGINE_H_
#define MSHADOW_EXPR_ENGINE_H_

#include "../tensor.h"

namespace mshadow {
namespace expr {

/*! \brief engine for expressions that are not elementwise; specialised per node type */
template <typename SV, typename RV, typename E, typename DType>
struct ExpComplexEngine {
  inline static void Eval(RV *dst, const E &exp);
};

template <typename SV, typename RV, typename DType>
struct ExpEngine {
  template <typename E>
  inline static void Eval(RV *dst, const Exp<E, DType, type::kMapper> &exp) {
    MapExp<SV>(dst, exp);
  }
  template <typename E>
  inline static void Eval(RV *dst, const Exp<E, DType, type::kChainer> &exp) {
    MapExp<SV>(dst, exp);
  }
  template <typename E>
  inline static void Eval(RV *dst, const Exp<E, DType, type::kRValue> &exp) {
    MapExp<SV>(dst, exp);
  }
  template <typename E>
  inline static void Eval(RV *dst, const Exp<E, DType, type::kComplex> &exp) {
    ExpComplexEngine<SV, RV, E, DType>::Eval(dst->ptrself(), exp.self());
  }
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXPR_ENGINE_H_
