/*
 * A caller-style program that runs every operation of the hot path in one chain, on one
 * stream: a convolution by unpack_patch2col + dot, bias by broadcast<1>, a user functor under
 * F<>, max pooling, reshape, a fully connected layer, Softmax in place; and back: sum_rows,
 * dot with transposed operands, unpool, sumall_except_dim<1>, pack_col2patch, scaled updates.
 * It is the network of the reference's guide/neuralnet/convnet.cu:81-122 (conv - maxpool -
 * fullc) written with the signatures the headers have today (6-argument pool, 7-argument
 * unpool and unpack_patch2col, 8-argument pack_col2patch), for any device tag, with the
 * containers padded as TensorContainer pads them by default and the same aliasing: the
 * activations are kept in a second container for the backward pass, the gradient of a layer
 * overwrites its activations, Softmax works in place. Two generalisations: the input may
 * have several channels, and the convolution may pad its input (pad(.) in front of
 * unpack_patch2col, crop(.) behind pack_col2patch), which is the geometry the patch kernels
 * are tuned for; with one channel and no padding the statements are those of the reference.
 *
 * Compiled three times from this one text - for Tensor<gpu> (cases.hip), for this backend's
 * Tensor<cpu> (tests/host/ext_cpu_cases.cc) and against the reference's own headers
 * (oracle/ref_driver.cc) - and compared tensor by tensor.
 */
#ifndef MSHADOW_AMD_CASES_CONV_NET_H_
#define MSHADOW_AMD_CASES_CONV_NET_H_

#include <mshadow/tensor.h>

namespace conv_net {

struct rectify {
  MSHADOW_XINLINE static float Map(float a) { return a < 0.0f ? 0.0f : a; }
};
struct rectify_grad {
  MSHADOW_XINLINE static float Map(float a) { return a > 0.0f ? 1.0f : 0.0f; }
};

/*! \brief sizes of the network; the derived ones follow convnet.cu:60-66 */
struct Geometry {
  int batch, in_channels, in_size, channels, ksize, kstride, pad, psize, num_out;
  int conv_out() const { return (in_size + 2 * pad - ksize) / kstride + 1; }
  int pool_out() const { return (conv_out() + 1 - psize) / psize; }
  int flat() const { return channels * pool_out() * pool_out(); }
  int patch() const { return in_channels * ksize * ksize; }
  int positions() const { return batch * conv_out() * conv_out(); }
};

/*! \brief the tensors a run hands back, each a dense host array (NULL: not wanted), in the
 *  order they come into being */
enum Kept {
  kColForward, kConvRaw, kHidden, kPooled, kLogits, kProbs,          // forward
  kGradOutBias, kGradOutWeight, kFlatGrad, kUnpooled, kHiddenGrad,   // backward
  kGradHiddenBias, kGradKernel, kColBackward, kInputGrad,
  kHiddenBias, kOutBias,                                             // after the update
  kKeptCount
};
/*! \brief elements of each of them */
inline size_t KeptSize(const Geometry &g, int which) {
  const size_t hidden = static_cast<size_t>(g.batch) * g.channels * g.conv_out() * g.conv_out();
  switch (which) {
    case kColForward: case kColBackward: return static_cast<size_t>(g.patch()) * g.positions();
    case kConvRaw: return static_cast<size_t>(g.channels) * g.positions();
    case kHidden: case kUnpooled: case kHiddenGrad: return hidden;
    case kPooled: case kFlatGrad: return static_cast<size_t>(g.batch) * g.flat();
    case kLogits: case kProbs: return static_cast<size_t>(g.batch) * g.num_out;
    case kGradOutBias: case kOutBias: return g.num_out;
    case kGradOutWeight: return static_cast<size_t>(g.flat()) * g.num_out;
    case kGradHiddenBias: case kHiddenBias: return g.channels;
    case kGradKernel: return static_cast<size_t>(g.channels) * g.patch();
    case kInputGrad: return static_cast<size_t>(g.batch) * g.in_channels * g.in_size * g.in_size;
    default: return 0;
  }
}

template <typename xpu>
class Net {
 public:
  typedef mshadow::Tensor<mshadow::cpu, 2, float> Host2;
  Net(mshadow::Stream<xpu> *stream, const Geometry &g, Host2 kernel0, Host2 weight0)
      : g_(g), stream_(stream) {
    using namespace mshadow;
    const index_t co = g.conv_out(), po = g.pool_out();
    Attach(&input_, Shape4(g.batch, g.in_channels, g.in_size, g.in_size));
    Attach(&hidden_, Shape4(g.batch, g.channels, co, co));
    Attach(&hidden_kept_, hidden_.shape_);
    Attach(&pooled_, Shape4(g.batch, g.channels, po, po));
    Attach(&pooled_kept_, pooled_.shape_);
    Attach(&flat_, Shape2(g.batch, g.flat()));
    Attach(&out_, Shape2(g.batch, g.num_out));
    Attach(&hidden_bias_, Shape1(g.channels));
    Attach(&grad_hidden_bias_, Shape1(g.channels));
    Attach(&out_bias_, Shape1(g.num_out));
    Attach(&grad_out_bias_, Shape1(g.num_out));
    Attach(&kernel_, Shape2(g.channels, g.patch()));
    Attach(&grad_kernel_, kernel_.shape_);
    Attach(&weight_, Shape2(g.flat(), g.num_out));
    Attach(&grad_weight_, weight_.shape_);
    Attach(&col_, Shape2(g.patch(), g.positions()));
    Attach(&conv_, Shape2(g.channels, g.positions()));
    hidden_bias_ = 0.0f;
    out_bias_ = 0.0f;
    Copy(kernel_, kernel0, stream_);
    Copy(weight_, weight0, stream_);
    for (int i = 0; i < kKeptCount; ++i) keep_[i] = NULL;
  }
  /*! \brief where the tensor `which` is to be copied when it comes into being */
  void Keep(int which, float *host) { keep_[which] = host; }

  void Forward(const mshadow::Tensor<mshadow::cpu, 4, float> &images, Host2 probs) {
    using namespace mshadow;
    using namespace mshadow::expr;
    Copy(input_, images, stream_);
    /* convolution: every patch unpacked into a column, one matrix product, and the
       (channel, image) order of the product swapped back */
    if (g_.pad == 0) {
      col_ = unpack_patch2col(input_, g_.ksize, g_.ksize, g_.kstride, g_.kstride, 1, 1);
    } else {
      col_ = unpack_patch2col(pad(input_, g_.pad), g_.ksize, g_.ksize, g_.kstride, g_.kstride, 1, 1);
    }
    Hand(kColForward, col_);
    conv_ = dot(kernel_, col_);
    Hand(kConvRaw, conv_);
    hidden_ = swapaxis<1, 0>(reshape(conv_, Shape4(g_.channels, g_.batch, g_.conv_out(), g_.conv_out())));
    hidden_ += broadcast<1>(hidden_bias_, hidden_.shape_);
    hidden_ = F<rectify>(hidden_);
    Copy(hidden_kept_, hidden_, stream_);
    Hand(kHidden, hidden_kept_);
    pooled_ = pool<red::maximum>(hidden_kept_, pooled_[0][0].shape_, g_.psize, g_.psize, g_.psize,
                                 g_.psize);
    Copy(pooled_kept_, pooled_, stream_);
    Hand(kPooled, pooled_kept_);
    flat_ = reshape(pooled_, flat_.shape_);
    out_ = dot(flat_, weight_);
    out_ += repmat(out_bias_, g_.batch);
    Hand(kLogits, out_);
    Softmax(out_, out_);
    Hand(kProbs, out_);
    Copy(probs, out_, stream_);
  }

  void Backprop(const Host2 &grad_out) {
    using namespace mshadow;
    using namespace mshadow::expr;
    Copy(out_, grad_out, stream_);
    grad_out_bias_ = sum_rows(out_);
    Hand(kGradOutBias, grad_out_bias_);
    grad_weight_ = dot(flat_.T(), out_);
    Hand(kGradOutWeight, grad_weight_);
    flat_ = dot(out_, weight_.T());
    Hand(kFlatGrad, flat_);
    pooled_ = reshape(flat_, pooled_.shape_);
    hidden_kept_ = unpool<red::maximum>(hidden_kept_, pooled_kept_, pooled_, g_.psize, g_.psize, g_.psize,
                                        g_.psize);
    Hand(kUnpooled, hidden_kept_);
    hidden_ = F<rectify_grad>(hidden_) * hidden_kept_;
    Hand(kHiddenGrad, hidden_);
    grad_hidden_bias_ = sumall_except_dim<1>(hidden_);
    Hand(kGradHiddenBias, grad_hidden_bias_);
    /* convolution backwards: the kernel's gradient, then the gradient of the input (not
       needed for a first layer, included as in the reference) */
    if (g_.pad == 0) {
      col_ = unpack_patch2col(input_, g_.ksize, g_.ksize, g_.kstride, g_.kstride, 1, 1);
    } else {
      col_ = unpack_patch2col(pad(input_, g_.pad), g_.ksize, g_.ksize, g_.kstride, g_.kstride, 1, 1);
    }
    conv_ = reshape(swapaxis<1, 0>(hidden_), conv_.shape_);
    grad_kernel_ = dot(conv_, col_.T());
    Hand(kGradKernel, grad_kernel_);
    col_ = dot(kernel_.T(), conv_);
    Hand(kColBackward, col_);
    if (g_.pad == 0) {
      input_ = pack_col2patch(col_, input_.shape_, g_.ksize, g_.ksize, g_.kstride, g_.kstride, 1, 1);
    } else {
      const index_t padded = g_.in_size + 2 * g_.pad;
      input_ = crop(pack_col2patch(col_, Shape4(g_.batch, g_.in_channels, padded, padded), g_.ksize,
                                   g_.ksize, g_.kstride, g_.kstride, 1, 1),
                    Shape2(g_.in_size, g_.in_size), g_.pad, g_.pad);
    }
    Hand(kInputGrad, input_);
  }

  void Update(float eta, float decay) {
    kernel_ -= eta * (decay * kernel_ + grad_kernel_);
    weight_ -= eta * (decay * weight_ + grad_weight_);
    hidden_bias_ -= eta * grad_hidden_bias_;
    out_bias_ -= eta * grad_out_bias_;
    Hand(kHiddenBias, hidden_bias_);
    Hand(kOutBias, out_bias_);
  }

  void Weights(Host2 kernel, Host2 weight) {
    mshadow::Copy(kernel, kernel_, stream_);
    mshadow::Copy(weight, weight_, stream_);
  }

 private:
  template <int dim>
  void Attach(mshadow::TensorContainer<xpu, dim, float> *t, mshadow::Shape<dim> shape) {
    t->set_stream(stream_);
    t->Resize(shape);
  }
  template <int dim>
  void Hand(int which, const mshadow::Tensor<xpu, dim, float> &t) {
    if (keep_[which] == NULL) return;
    mshadow::Copy(mshadow::Tensor<mshadow::cpu, dim, float>(keep_[which], t.shape_), t, stream_);
  }

  Geometry g_;
  mshadow::Stream<xpu> *stream_;
  float *keep_[kKeptCount];
  mshadow::TensorContainer<xpu, 4, float> input_, hidden_, hidden_kept_, pooled_, pooled_kept_;
  mshadow::TensorContainer<xpu, 2, float> flat_, out_, col_, conv_;
  mshadow::TensorContainer<xpu, 1, float> hidden_bias_, out_bias_, grad_hidden_bias_, grad_out_bias_;
  mshadow::TensorContainer<xpu, 2, float> kernel_, weight_, grad_kernel_, grad_weight_;
};

/*!
 * \brief `steps` rounds of forward, backward and update on one batch; every pointer is host
 *  memory. The gradient that enters the backward pass is made on the host as in the
 *  reference's main loop (convnet.cu:252-259): probs - onehot(label), divided by the batch
 *  size - or, if `fixed_grad` is given, is that array on every round (values chosen by a test).
 * \param kernel, weight initial values on entry, trained values on return
 * \param keep kKeptCount host arrays (or NULL each) for the tensors of the last round
 */
template <typename xpu>
inline void Train(mshadow::Stream<xpu> *stream, const Geometry &g, int steps, float eta, float decay,
                  const float *images, const float *labels, const float *fixed_grad, float *kernel,
                  float *weight, float *const *keep) {
  using namespace mshadow;
  Tensor<cpu, 2, float> k0(kernel, Shape2(g.channels, g.patch()));
  Tensor<cpu, 2, float> w0(weight, Shape2(g.flat(), g.num_out));
  Tensor<cpu, 4, float> x(const_cast<float *>(images), Shape4(g.batch, g.in_channels, g.in_size, g.in_size));
  TensorContainer<cpu, 2, float> pred(Shape2(g.batch, g.num_out));
  Net<xpu> net(stream, g, k0, w0);
  for (int s = 0; s < steps; ++s) {
    if (s + 1 == steps && keep != NULL) {
      for (int i = 0; i < kKeptCount; ++i) net.Keep(i, keep[i]);
    }
    net.Forward(x, pred);
    if (stream != NULL) stream->Wait();
    if (fixed_grad != NULL) {
      Copy(pred, Tensor<cpu, 2, float>(const_cast<float *>(fixed_grad), pred.shape_));
    } else {
      for (int b = 0; b < g.batch; ++b) pred[b][static_cast<index_t>(labels[b])] -= 1.0f;
      pred *= 1.0f / g.batch;
    }
    net.Backprop(pred);
    net.Update(eta, decay);
  }
  net.Weights(k0, w0);
  if (stream != NULL) stream->Wait();
}

/*!
 * \brief the convolution pair alone for any element type (binary16 is what the patch kernels
 *  are tuned for): out = conv(image, kernel) through unpack_patch2col, and the gradient of
 *  the image for a given gradient of out through pack_col2patch. The two matrix products run
 *  in float (tcast in, tcast out): the stand-alone reference has no product for 16-bit
 *  elements. Every pointer is host memory of DType.
 */
template <typename xpu, typename DType>
inline void ConvPair(mshadow::Stream<xpu> *stream, const Geometry &g, const DType *image,
                     const DType *kernel, const DType *grad_out, DType *col_forward, DType *out,
                     DType *col_backward, DType *image_grad) {
  using namespace mshadow;
  using namespace mshadow::expr;
  const index_t co = g.conv_out(), padded = g.in_size + 2 * g.pad;
  const Shape<4> in_shape = Shape4(g.batch, g.in_channels, g.in_size, g.in_size);
  const Shape<4> out_shape = Shape4(g.batch, g.channels, co, co);
  const Shape<2> col_shape = Shape2(g.patch(), g.positions());
  const Shape<2> conv_shape = Shape2(g.channels, g.positions());
  TensorContainer<xpu, 4, DType> in, gout, result;
  TensorContainer<xpu, 2, DType> k, col, conv;
  TensorContainer<xpu, 2, float> kf, colf, convf;
  in.set_stream(stream), gout.set_stream(stream), result.set_stream(stream), k.set_stream(stream);
  col.set_stream(stream), conv.set_stream(stream), kf.set_stream(stream), colf.set_stream(stream);
  convf.set_stream(stream);
  in.Resize(in_shape), gout.Resize(out_shape), result.Resize(out_shape);
  k.Resize(Shape2(g.channels, g.patch())), col.Resize(col_shape), conv.Resize(conv_shape);
  kf.Resize(k.shape_), colf.Resize(col_shape), convf.Resize(conv_shape);
  Copy(in, Tensor<cpu, 4, DType>(const_cast<DType *>(image), in_shape), stream);
  Copy(k, Tensor<cpu, 2, DType>(const_cast<DType *>(kernel), k.shape_), stream);
  Copy(gout, Tensor<cpu, 4, DType>(const_cast<DType *>(grad_out), out_shape), stream);
  kf = tcast<float>(k);
  col = unpack_patch2col(pad(in, g.pad), g.ksize, g.ksize, g.kstride, g.kstride, 1, 1);
  Copy(Tensor<cpu, 2, DType>(col_forward, col_shape), col, stream);
  colf = tcast<float>(col);
  convf = dot(kf, colf);
  conv = tcast<DType>(convf);
  result = swapaxis<1, 0>(reshape(conv, Shape4(g.channels, g.batch, co, co)));
  Copy(Tensor<cpu, 4, DType>(out, out_shape), result, stream);
  conv = reshape(swapaxis<1, 0>(gout), conv_shape);
  convf = tcast<float>(conv);
  colf = dot(kf.T(), convf);
  col = tcast<DType>(colf);
  Copy(Tensor<cpu, 2, DType>(col_backward, col_shape), col, stream);
  in = crop(pack_col2patch(col, Shape4(g.batch, g.in_channels, padded, padded), g.ksize, g.ksize,
                           g.kstride, g.kstride, 1, 1),
            Shape2(g.in_size, g.in_size), g.pad, g.pad);
  Copy(Tensor<cpu, 4, DType>(image_grad, in_shape), in, stream);
  if (stream != NULL) stream->Wait();
}

}  // namespace conv_net
#endif  // MSHADOW_AMD_CASES_CONV_NET_H_
