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

namespace reduce_detail {
/*! \brief the node type for keeping dimension `dimkeep` (counted from the front) of SrcExp */
template <int dimkeep, typename Reducer, typename SrcExp, typename DType>
struct NodeFor {
  typedef ReduceTo1DExp<SrcExp, DType, Reducer, ExpInfo<SrcExp>::kDim - dimkeep> Type;
  inline static Type Make(const SrcExp &src) { return Type(src, DType(1)); }
};
/*! \brief which device function evaluates the node: the kept dimension is the last one
 *  (every output is a chain over the rows) or any other (two-level reduction) */
template <bool kKeepsLast>
struct Evaluate {
  template <typename SV, typename Reducer, int dimkeep, typename Dst, typename SrcExp, typename DType>
  inline static void Run(Dst *dst, const SrcExp &src, DType scale) {
    MapReduceKeepHighDim<SV, Reducer, dimkeep>(dst, src, scale);
  }
};
template <>
struct Evaluate<true> {
  template <typename SV, typename Reducer, int dimkeep, typename Dst, typename SrcExp, typename DType>
  inline static void Run(Dst *dst, const SrcExp &src, DType scale) {
    MapReduceKeepLowest<SV, Reducer>(dst, src, scale);
  }
};
}  // namespace reduce_detail

template <int dimkeep, typename Reducer, typename SrcExp, typename DType, int etype>
inline typename reduce_detail::NodeFor<dimkeep, Reducer, SrcExp, DType>::Type reduce_except_dim(
    const Exp<SrcExp, DType, etype> &exp) {
  return reduce_detail::NodeFor<dimkeep, Reducer, SrcExp, DType>::Make(exp.self());
}
template <int dimkeep, typename SrcExp, typename DType, int etype>
inline typename reduce_detail::NodeFor<dimkeep, red::sum, SrcExp, DType>::Type sumall_except_dim(
    const Exp<SrcExp, DType, etype> &exp) {
  return reduce_except_dim<dimkeep, red::sum>(exp);
}
/*! \brief column sums of a matrix */
template <typename SrcExp, typename DType, int etype>
inline ReduceTo1DExp<SrcExp, DType, red::sum, 1> sum_rows(const Exp<SrcExp, DType, etype> &exp) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim == 2>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return sumall_except_dim<1>(exp);
}

/*! \brief dst [sv] node: one engine for every kept dimension */
template <typename SV, typename Device, typename DType, typename SrcExp, typename Reducer,
          int m_dimkeep>
struct ExpComplexEngine<SV, Tensor<Device, 1, DType>,
                        ReduceTo1DExp<SrcExp, DType, Reducer, m_dimkeep>, DType> {
  inline static void Eval(Tensor<Device, 1, DType> *dst,
                          const ReduceTo1DExp<SrcExp, DType, Reducer, m_dimkeep> &exp) {
    reduce_detail::Evaluate<m_dimkeep == 1>::template Run<SV, Reducer,
                                                          ExpInfo<SrcExp>::kDim - m_dimkeep>(
        dst, exp.src_, exp.scale_);
  }
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_REDUCETO1D_H_
