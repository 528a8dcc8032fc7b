/*
 * chpool<Reducer>(src, nsize[, stride, pad]) and ch_unpool<Reducer>(src, pooled, grad, ...):
 * reduction over neighbouring channels (the third dimension from the end) and its
 * gradient, the building blocks of local response normalisation.
 *
 * Behaviour restates mshadow/extension/channel_pool.h:21-108 and
 * channel_unpool.h:21-137 of the reference, including two properties a caller may rely
 * on without knowing:
 *  - the pooled channel count is (C - nsize + 2 pad + 1) / stride (floor), and the
 *    window of pooled channel c is [c stride - pad, c stride - pad + nsize) cut at 0
 *    below and at the POOLED channel count above (not at C);
 *  - ch_unpool visits, for source channel c, the pooled channels from
 *    (c - (nsize - pad) + stride) / stride (0 if c < nsize - pad) up to
 *    (c + pad + stride) / stride, cut at the SOURCE channel count, ascending, and adds
 *    PartialGrad(src, pooled) * grad.
 * With the defaults (stride 1, pad nsize / 2, odd nsize) both counts are C and neither
 * cut matters. Where those cuts would let a window run past the tensor it reads (the
 * reference then reads whatever follows in memory), the window here also ends at that
 * tensor's channel count. Channels are reduced in ascending order from
 * Reducer::SetInitValue.
 */
#ifndef MSHADOW_EXT_CHANNELS_H_
#define MSHADOW_EXT_CHANNELS_H_

#include "../core/fastdiv.h"
#include "../tensor.h"

namespace mshadow {
namespace expr {

template <typename Reducer, typename SrcExp, typename DType, int srcdim>
struct ChannelPoolingExp
    : public MakeTensorExp<ChannelPoolingExp<Reducer, SrcExp, DType, srcdim>, SrcExp, srcdim,
                           DType> {
  const SrcExp &src_;
  index_t nsize_, stride_, pad_;
  index_t src_channel_;
  ChannelPoolingExp(const SrcExp &src, index_t nsize, index_t stride, index_t pad)
      : src_(src), nsize_(nsize), stride_(stride), pad_(pad) {
    this->shape_ = ShapeCheck<srcdim, SrcExp>::Check(src_);
    src_channel_ = this->shape_[srcdim - 3];
    CHECK_GE(src_channel_, nsize_) << "chpool: local size must be smaller than nchannels";
    this->shape_[srcdim - 3] = (src_channel_ - nsize + pad * 2 + 1) / stride;
  }
};

template <typename Reducer, typename SrcExp, typename DType, int etype>
inline ChannelPoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim> chpool(
    const Exp<SrcExp, DType, etype> &src, index_t nsize) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 3>::Error_Expression_Does_Not_Meet_Dimension_Req();
  CHECK_EQ(nsize % 2, 1U) << "chpool: if no pad is specified, local size must be odd";
  return ChannelPoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), nsize, 1,
                                                                          nsize / 2);
}
template <typename Reducer, typename SrcExp, typename DType, int etype>
inline ChannelPoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim> chpool(
    const Exp<SrcExp, DType, etype> &src, index_t nsize, index_t stride, index_t pad) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 3>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return ChannelPoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim>(src.self(), nsize,
                                                                          stride, pad);
}

template <typename Reducer, typename SrcExp, typename DType, int srcdim>
struct Plan<ChannelPoolingExp<Reducer, SrcExp, DType, srcdim>, DType> {
 public:
  explicit Plan(const ChannelPoolingExp<Reducer, SrcExp, DType, srcdim> &e)
      : src_(MakePlan(e.src_)), channel_(e.shape_[srcdim - 3]), height_(e.shape_[srcdim - 2]),
        nsize_(e.nsize_), stride_(e.stride_), pad_(e.pad_), src_channel_(e.src_channel_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const index_t plane = height_.Div(i);  // (image, pooled channel)
    const index_t y = i - plane * height_.div;
    const index_t n = channel_.Div(plane);
    const index_t c = plane - n * channel_.div;
    const index_t first = c * stride_ < pad_ ? 0 : c * stride_ - pad_;
    index_t last = c * stride_ - pad_ + nsize_;
    if (last > channel_.div) last = channel_.div;
    if (last > src_channel_) last = src_channel_;
    DType res;
    Reducer::SetInitValue(res);
    /* four channels fetched before they are reduced, in channel order either way: the loads
       do not wait for each other */
    const index_t step = height_.div;
    index_t row = (n * src_channel_ + first) * step + y;
    index_t cc = first;
    for (; cc + 4 <= last; cc += 4, row += 4 * step) {
      const DType v0 = src_.Eval(row, j), v1 = src_.Eval(row + step, j),
                  v2 = src_.Eval(row + 2 * step, j), v3 = src_.Eval(row + 3 * step, j);
      Reducer::Reduce(res, v0);
      Reducer::Reduce(res, v1);
      Reducer::Reduce(res, v2);
      Reducer::Reduce(res, v3);
    }
    for (; cc < last; ++cc, row += step) Reducer::Reduce(res, src_.Eval(row, j));
    return res;
  }
  /* the window runs over rows of the source at the same column: N adjacent columns at once */
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t i, index_t j) const {
    const index_t plane = height_.Div(i);
    const index_t y = i - plane * height_.div;
    const index_t n = channel_.Div(plane);
    const index_t c = plane - n * channel_.div;
    const index_t first = c * stride_ < pad_ ? 0 : c * stride_ - pad_;
    index_t last = c * stride_ - pad_ + nsize_;
    if (last > channel_.div) last = channel_.div;
    if (last > src_channel_) last = src_channel_;
    /* the usual window sizes as straight-line code: all fetches of a window (and of the other
       packs the calling thread evaluates) are in flight together */
    if (nsize_ == 5) return FixedWindow<5, N>(n, c, y, j, last);
    if (nsize_ == 3) return FixedWindow<3, N>(n, c, y, j, last);
    Pack<DType, N> res;
#pragma unroll
    for (int k = 0; k < N; ++k) Reducer::SetInitValue(res.v[k]);
    const index_t step = height_.div;
    index_t row = (n * src_channel_ + first) * step + y;
    index_t cc = first;
    /* neighbouring windows read the same rows again: ordinary (cached) loads */
    for (; cc + 4 <= last; cc += 4, row += 4 * step) {
      const Pack<DType, N> v0 = src_.template EvalPack<N, false>(row, j),
                           v1 = src_.template EvalPack<N, false>(row + step, j),
                           v2 = src_.template EvalPack<N, false>(row + 2 * step, j),
                           v3 = src_.template EvalPack<N, false>(row + 3 * step, j);
#pragma unroll
      for (int k = 0; k < N; ++k) {
        Reducer::Reduce(res.v[k], v0.v[k]);
        Reducer::Reduce(res.v[k], v1.v[k]);
        Reducer::Reduce(res.v[k], v2.v[k]);
        Reducer::Reduce(res.v[k], v3.v[k]);
      }
    }
    for (; cc < last; ++cc, row += step) {
      const Pack<DType, N> v = src_.template EvalPack<N, false>(row, j);
#pragma unroll
      for (int k = 0; k < N; ++k) Reducer::Reduce(res.v[k], v.v[k]);
    }
    return res;
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    *flat = false;
    bool ignored = true;
    return src_.PackReady(n, cols, &ignored);
  }
  /*! \brief windows of neighbouring pooled channels overlap in all but `stride` planes */
  inline index_t PlaneRows() const { return nsize_ > stride_ ? height_.div : 0; }
  static const bool kPlaneWindow = kPackable;
  /*! \brief the same place (y, j) of K planes dy rows apart, starting at row i0. When these
   *  are K consecutive pooled channels of one image with windows one channel apart, the
   *  K + nsize - 1 source channels under them are fetched once and every window is reduced
   *  from registers, in channel order as always. */
  template <int N, bool STREAM, int K>
  MSHADOW_XINLINE void EvalPackRun(index_t i0, index_t dy, index_t j, Pack<DType, N> *out) const {
    const index_t plane = height_.Div(i0);
    const index_t y = i0 - plane * height_.div;
    const index_t n = channel_.Div(plane);
    const index_t c0 = plane - n * channel_.div;
    if (dy == height_.div && stride_ == 1 && c0 + K <= channel_.div) {
      if (nsize_ == 5) return SharedWindows<5, N, K>(n, c0, y, j, out);
      if (nsize_ == 3) return SharedWindows<3, N, K>(n, c0, y, j, out);
    }
#pragma unroll
    for (int u = 0; u < K; ++u) out[u] = this->template EvalPack<N, STREAM>(i0 + u * dy, j);
  }

 private:
  template <int W, int N, int K>
  MSHADOW_XINLINE void SharedWindows(index_t n, index_t c0, index_t y, index_t j,
                                     Pack<DType, N> *out) const {
    const index_t step = height_.div;
    const index_t start = c0 - pad_;  // may be negative: those positions are skipped
    const index_t limit = channel_.div < src_channel_ ? channel_.div : src_channel_;
    Pack<DType, N> v[K + W - 1];
    bool inside[K + W - 1];
#pragma unroll
    for (int k = 0; k < K + W - 1; ++k) {
      const index_t cc = start + k;
      inside[k] = cc >= 0 && cc < limit;
      const index_t safe = inside[k] ? cc : 0;
      v[k] = src_.template EvalPack<N, false>((n * src_channel_ + safe) * step + y, j);
    }
#pragma unroll
    for (int u = 0; u < K; ++u) {
#pragma unroll
      for (int e = 0; e < N; ++e) Reducer::SetInitValue(out[u].v[e]);
#pragma unroll
      for (int k = 0; k < W; ++k) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
          DType with = out[u].v[e];
          Reducer::Reduce(with, v[u + k].v[e]);
          out[u].v[e] = inside[u + k] ? with : out[u].v[e];
        }
      }
    }
  }
  /*! \brief a window of K channels starting at c * stride - pad and ending before `last`:
   *  every position is fetched (a position outside the window re-reads the pooled channel's
   *  own row index clamped into the source, and is not reduced), then reduced in channel order */
  template <int K, int N>
  MSHADOW_XINLINE Pack<DType, N> FixedWindow(index_t n, index_t c, index_t y, index_t j,
                                             index_t last) const {
    const index_t step = height_.div;
    const index_t start = c * stride_ - pad_;  // may be negative: those positions are skipped
    Pack<DType, N> v[K];
    bool inside[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const index_t cc = start + k;
      inside[k] = cc >= 0 && cc < last;
      const index_t safe = inside[k] ? cc : 0;
      v[k] = src_.template EvalPack<N, false>((n * src_channel_ + safe) * step + y, j);
    }
    Pack<DType, N> res;
#pragma unroll
    for (int e = 0; e < N; ++e) Reducer::SetInitValue(res.v[e]);
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
      for (int e = 0; e < N; ++e) {
        DType with = res.v[e];
        Reducer::Reduce(with, v[k].v[e]);
        res.v[e] = inside[k] ? with : res.v[e];
      }
    }
    return res;
  }
  Plan<SrcExp, DType> src_;
  const FastDivU32 channel_, height_;
  const index_t nsize_, stride_, pad_, src_channel_;
};

template <typename Reducer, typename SrcExp, typename DType, int srcdim>
struct ChannelUnpoolingExp
    : public MakeTensorExp<ChannelUnpoolingExp<Reducer, SrcExp, DType, srcdim>, SrcExp, srcdim,
                           DType> {
  const SrcExp &data_src_;
  const SrcExp &data_pooled_;
  const SrcExp &grad_pooled_;
  index_t pchannel_;
  index_t nsize_, kstride_, pad_;
  ChannelUnpoolingExp(const SrcExp &data_src, const SrcExp &data_pooled,
                      const SrcExp &grad_pooled, index_t nsize, index_t kstride, index_t pad)
      : data_src_(data_src), data_pooled_(data_pooled), grad_pooled_(grad_pooled), nsize_(nsize),
        kstride_(kstride), pad_(pad) {
    Shape<srcdim> pshape = ShapeCheck<srcdim, SrcExp>::Check(grad_pooled);
    CHECK_EQ(pshape, (ShapeCheck<srcdim, SrcExp>::Check(data_pooled)))
        << "ChannelUnPoolingExp: data and grad shape mismatch";
    Shape<srcdim> sshape = ShapeCheck<srcdim, SrcExp>::Check(data_src);
    /* every dimension but the second must agree (as the reference checks it) */
    for (int k = 0; k < srcdim; ++k) {
      if (k == 1) continue;
      CHECK_EQ(pshape[k], sshape[k])
          << "ChannelUnPoolingExp: pooled tensor and src tensor shape mismatch" << pshape[k]
          << " vs " << sshape[k];
    }
    pchannel_ = pshape[1];
    this->shape_ = sshape;
  }
};

template <typename Reducer, typename SrcExp, typename DType, int etype>
inline ChannelUnpoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim> ch_unpool(
    const Exp<SrcExp, DType, etype> &data_src, const Exp<SrcExp, DType, etype> &data_pooled,
    const Exp<SrcExp, DType, etype> &grad_pooled, index_t nsize, index_t stride, index_t pad) {
  TypeCheckPass<ExpInfo<SrcExp>::kDim >= 3>::Error_Expression_Does_Not_Meet_Dimension_Req();
  return ChannelUnpoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim>(
      data_src.self(), data_pooled.self(), grad_pooled.self(), nsize, stride, pad);
}
template <typename Reducer, typename SrcExp, typename DType, int etype>
inline ChannelUnpoolingExp<Reducer, SrcExp, DType, ExpInfo<SrcExp>::kDim> ch_unpool(
    const Exp<SrcExp, DType, etype> &data_src, const Exp<SrcExp, DType, etype> &data_pooled,
    const Exp<SrcExp, DType, etype> &grad_pooled, index_t nsize) {
  return ch_unpool<Reducer>(data_src, data_pooled, grad_pooled, nsize, 1, nsize / 2);
}

template <typename Reducer, typename SrcExp, typename DType, int srcdim>
struct Plan<ChannelUnpoolingExp<Reducer, SrcExp, DType, srcdim>, DType> {
 public:
  explicit Plan(const ChannelUnpoolingExp<Reducer, SrcExp, DType, srcdim> &e)
      : src_(MakePlan(e.data_src_)), pooled_(MakePlan(e.data_pooled_)),
        grad_(MakePlan(e.grad_pooled_)), channel_(e.shape_[srcdim - 3]),
        height_(e.shape_[srcdim - 2]), pchannel_(e.pchannel_), nsize_(e.nsize_),
        stride_(e.kstride_), pad_(e.pad_) {}
  MSHADOW_XINLINE DType Eval(index_t i, index_t j) const {
    const DType vsrc = src_.Eval(i, j);
    const index_t plane = height_.Div(i);  // (image, source channel)
    const index_t y = i - plane * height_.div;
    const index_t n = channel_.Div(plane);
    const index_t c = plane - n * channel_.div;
    const index_t reach = nsize_ - pad_;
    const index_t first = c < reach ? 0 : stride_.Div(c - reach + stride_.div);
    index_t last = stride_.Div(c + pad_ + stride_.div);
    if (last > channel_.div) last = channel_.div;
    if (last > pchannel_) last = pchannel_;
    DType val = static_cast<DType>(0);
    for (index_t cc = first; cc < last; ++cc) {
      const index_t row = (n * pchannel_ + cc) * height_.div + y;
      val += Reducer::PartialGrad(vsrc, pooled_.Eval(row, j)) * grad_.Eval(row, j);
    }
    return val;
  }
  static const bool kPackable = plan_detail::Packable<Plan<SrcExp, DType> >::value;
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t i, index_t j) const {
    const Pack<DType, N> vsrc = src_.template EvalPack<N, STREAM>(i, j);
    const index_t plane = height_.Div(i);
    const index_t y = i - plane * height_.div;
    const index_t n = channel_.Div(plane);
    const index_t c = plane - n * channel_.div;
    const index_t reach = nsize_ - pad_;
    const index_t first = c < reach ? 0 : stride_.Div(c - reach + stride_.div);
    index_t last = stride_.Div(c + pad_ + stride_.div);
    if (last > channel_.div) last = channel_.div;
    if (last > pchannel_) last = pchannel_;
    Pack<DType, N> val;
#pragma unroll
    for (int k = 0; k < N; ++k) val.v[k] = static_cast<DType>(0);
    index_t row = (n * pchannel_ + first) * height_.div + y;
    for (index_t cc = first; cc < last; ++cc, row += height_.div) {
      const Pack<DType, N> p = pooled_.template EvalPack<N, false>(row, j),
                           g = grad_.template EvalPack<N, false>(row, j);
#pragma unroll
      for (int k = 0; k < N; ++k) val.v[k] += Reducer::PartialGrad(vsrc.v[k], p.v[k]) * g.v[k];
    }
    return val;
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    *flat = false;
    bool ignored = true;
    return src_.PackReady(n, cols, &ignored) && pooled_.PackReady(n, cols, &ignored) &&
           grad_.PackReady(n, cols, &ignored);
  }

 private:
  Plan<SrcExp, DType> src_, pooled_, grad_;
  const FastDivU32 channel_, height_;
  const index_t pchannel_, nsize_;
  const FastDivU32 stride_;
  const index_t pad_;
};

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXT_CHANNELS_H_
