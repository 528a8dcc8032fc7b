/*
 * A caller-style program that strings the pieces together: a two-layer perceptron trained by
 * plain gradient descent on one batch, written once for any device tag. It uses what the
 * reference's guide/neuralnet/nnet.cu uses - TensorContainer, Copy between devices, dot with
 * transposed operands, repmat, a user functor under F<>, Softmax, sum_rows, scaled updates -
 * with the signatures the headers have today (SoftmaxGrad instead of a host-side subtraction).
 * Compiled for gpu in cases.hip and for cpu in tests/host; the test compares both with a
 * float64 model.
 */
#ifndef MSHADOW_AMD_CASES_TWO_LAYER_NET_H_
#define MSHADOW_AMD_CASES_TWO_LAYER_NET_H_

#include <mshadow/tensor.h>

#include "portable_math.h"

namespace two_layer_net {

struct logistic {
  MSHADOW_XINLINE static float Map(float a) { return pmath_sigmoid(a); }
};

/*!
 * \brief `steps` full-batch updates of  p = softmax(logistic(x W1 + b1) W2 + b2)  towards
 *  the labels, biases starting at zero; every argument is host memory
 * \param w1, w2 initial weights on entry, trained weights on return
 * \param probs the forward pass of the last step (before its update)
 */
template <typename xpu>
inline void Train(mshadow::Stream<xpu> *stream, int steps, float eta, float decay,
                  mshadow::Tensor<mshadow::cpu, 2, float> x,
                  mshadow::Tensor<mshadow::cpu, 1, float> label,
                  mshadow::Tensor<mshadow::cpu, 2, float> w1,
                  mshadow::Tensor<mshadow::cpu, 2, float> w2,
                  mshadow::Tensor<mshadow::cpu, 2, float> probs) {
  using namespace mshadow;
  using namespace mshadow::expr;
  const index_t batch = x.size(0), hidden = w1.size(1), classes = w2.size(1);
  TensorContainer<xpu, 2, float> in(x.shape_), act(Shape2(batch, hidden)),
      act_grad(Shape2(batch, hidden)), out(Shape2(batch, classes)), W1(w1.shape_), W2(w2.shape_),
      gW1(w1.shape_), gW2(w2.shape_);
  TensorContainer<xpu, 1, float> b1(Shape1(hidden)), b2(Shape1(classes)), gb1(Shape1(hidden)),
      gb2(Shape1(classes)), target(label.shape_);
  in.set_stream(stream), act.set_stream(stream), act_grad.set_stream(stream);
  out.set_stream(stream), W1.set_stream(stream), W2.set_stream(stream);
  gW1.set_stream(stream), gW2.set_stream(stream), b1.set_stream(stream), b2.set_stream(stream);
  gb1.set_stream(stream), gb2.set_stream(stream), target.set_stream(stream);
  Copy(in, x, stream);
  Copy(W1, w1, stream);
  Copy(W2, w2, stream);
  Copy(target, label, stream);
  b1 = 0.0f;
  b2 = 0.0f;
  for (int s = 0; s < steps; ++s) {
    act = dot(in, W1);
    act += repmat(b1, batch);
    act = F<logistic>(act);
    out = dot(act, W2);
    out += repmat(b2, batch);
    Softmax(out, out);
    if (s + 1 == steps) Copy(probs, out, stream);
    SoftmaxGrad(out, out, target);  // d(loss) / d(logits) of the summed cross entropy
    out *= 1.0f / batch;
    gb2 = sum_rows(out);
    gW2 = dot(act.T(), out);
    act_grad = dot(out, W2.T());
    act_grad = act * (1.0f - act) * act_grad;
    gb1 = sum_rows(act_grad);
    gW1 = dot(in.T(), act_grad);
    W1 -= eta * (decay * W1 + gW1);
    W2 -= eta * (decay * W2 + gW2);
    b1 -= eta * gb1;
    b2 -= eta * gb2;
  }
  Copy(w1, W1, stream);
  Copy(w2, W2, stream);
  if (stream != NULL) stream->Wait();
}

}  // namespace two_layer_net
#endif  // MSHADOW_AMD_CASES_TWO_LAYER_NET_H_
