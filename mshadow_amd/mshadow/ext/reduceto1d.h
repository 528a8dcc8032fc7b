/*
 * Reduce an expression to a 1-D tensor, keeping one dimension:
 *   dst [sv] [scale *] sumall_except_dim<k>(src)
 *   dst [sv] [scale *] reduce_except_dim<k, Reducer>(src)
 *   dst [sv] [scale *] sum_rows(src)            (2-D src, keeps the columns)
 * Node and entry points per mshadow/extension/reduceto1d.h:22-101 of the reference.
 * Keeping the last dimension dispatches to MapReduceKeepLowest, any other to
 * MapReduceKeepHighDim.
 */
#ifndef MSHADOW_EXT_REDUCETO1D_H_
#define MSHADOW_EXT_REDUCETO1D_H_

#include "../tensor.h"

namespace mshadow {
namespace expr {

/*! \brief m_dimkeep counts the kept dimension from the end: 1 is the last one */
template <typename SrcExp, typename DType, typename Reducer, int m_dimkeep>
struct ReduceTo1DExp
    : public Exp<ReduceTo1DExp<SrcExp, DType, Reducer, m_dimkeep>, DType, type::kComplex> {
  const SrcExp &src_;
  DType scale_;
  ReduceTo1DExp(const SrcExp &src, DType scale) : src_(src), scale_(scale) {}
};

template <int dimkeep, typename SrcExp, typename DType, int etype>
inline ReduceTo1DExp<SrcExp, DType, red::sum, ExpInfo<SrcExp>::kDim - dimkeep> sumall_except_dim(
    const Exp<SrcExp, DType, etype> &exp) {
  return ReduceTo1DExp<SrcExp, DType, red::sum, ExpInfo<SrcExp>::kDim - dimkeep>(exp.self(),
                                                                                  DType(1));
}
template <int dimkeep, typename Reducer, typename SrcExp, typename DType, int etype>
inline ReduceTo1DExp<SrcExp, DType, Reducer, ExpInfo<SrcExp>::kDim - dimkeep> reduce_except_dim(
    const Exp<SrcExp, DType, etype> &exp) {
  return ReduceTo1DExp<SrcExp, DType, Reducer, ExpInfo<SrcExp>::kDim - dimkeep>(exp.self(),
                                                                                 DType(1));
}
template <typename SrcExp, typename DType, int etype>
inline ReduceTo1DExp<SrcExp, DType, red::sum, 1> sum_rows(const Exp<SrcExp, DType, etype> &exp) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim == 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return sumall_except_dim<1>(exp);
}

template <typename SV, typename Device, typename DType, typename SrcExp, typename Reducer,
          int m_dimkeep>
struct ExpComplexEngine<SV, Tensor<Device, 1, DType>,
                        ReduceTo1DExp<SrcExp, DType, Reducer, m_dimkeep>, DType> {
  static const int dimkeep = ExpInfo<SrcExp>::kDim - m_dimkeep;
  inline static void Eval(Tensor<Device, 1, DType> *dst,
                          const ReduceTo1DExp<SrcExp, DType, Reducer, m_dimkeep> &exp) {
    TypeCheckPass<m_dimkeep != 1>::Error_Expression_Does_Not_Meet_Dimension_Req();
    MapReduceKeepHighDim<SV, Reducer, dimkeep>(dst, exp.src_, exp.scale_);
  }
};
template <typename SV, typename Device, typename DType, typename SrcExp, typename Reducer>
struct ExpComplexEngine<SV, Tensor<Device, 1, DType>, ReduceTo1DExp<SrcExp, DType, Reducer, 1>,
                        DType> {
  inline static void Eval(Tensor<Device, 1, DType> *dst,
                          const ReduceTo1DExp<SrcExp, DType, Reducer, 1> &exp) {
    MapReduceKeepLowest<SV, Reducer>(dst, exp.src_, exp.scale_);
  }
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_REDUCETO1D_H_
