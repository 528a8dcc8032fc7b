// The extension expressions of mshadow_amd/cases/extension_cases.inc evaluated on
// Tensor<cpu> of this backend's headers (plain g++, no GPU): built as a small shared
// library by tests/test_extensions.py and compared with numpy there.
#include <mshadow/tensor.h>
#include <mshadow/random.h>

#include "../../mshadow_amd/cases/portable_math.h"
#include "../../mshadow_amd/cases/two_layer_net.h"
#include "../../mshadow_amd/cases/conv_net.h"

using namespace mshadow;
using namespace mshadow::expr;

namespace {
template <int dim>
Tensor<cpu, dim, float> View(const float *p, Shape<dim> shape) {
  return Tensor<cpu, dim, float>(const_cast<float *>(p), shape);
}
}  // namespace

/* caller-side functor of the product cases, same arithmetic as the device build */
struct sigmoid {
  MSHADOW_XINLINE static float Map(float a) { return pmath_sigmoid(a); }
};

/* caller-side functor of the extension cases (local response normalisation squares its input) */
struct square_of {
  MSHADOW_XINLINE static float Map(float a) { return a * a; }
};

extern "C" int host_extensions_f32(int op, float *out, const float *a, const float *b,
                                   const float *c, int n, int ch, int h, int w, int p0, int p1,
                                   int p2) {
  try {
#define TENSOR(dim) Tensor<cpu, dim, float>
#define V1(p, len) View(p, Shape1(len))
#define V2(p, d0, d1) View(p, Shape2(d0, d1))
#define V3(p, d0, d1, d2) View(p, Shape3(d0, d1, d2))
#define V4(p, d0, d1, d2, d3) View(p, Shape4(d0, d1, d2, d3))
#define V4S(p, d0, d1, d2, d3, pitch) \
  Tensor<cpu, 4, float>(const_cast<float *>(p), Shape4(d0, d1, d2, d3), pitch, NULL)
#include "../../mshadow_amd/cases/extension_cases.inc"
#undef TENSOR
#undef V1
#undef V2
#undef V3
#undef V4S
#undef V4
  } catch (const std::exception &e) {
    fprintf(stderr, "%s\n", e.what());
    return 1;
  }
  return 0;
}

extern "C" int host_random_f32(int op, int seed, float *out, int n, float p0, float p1) {
  try {
#include "../../mshadow_amd/cases/random_cases.inc"
  } catch (const std::exception &e) {
    fprintf(stderr, "%s\n", e.what());
    return 1;
  }
  return 0;
}

extern "C" int host_dot_f32(int op, float *out, const float *a, const float *b, int m, int k,
                            int n, int batch) {
  try {
#define XPU cpu
#define STREAM static_cast<Stream<cpu> *>(NULL)
#define TENSOR(dim) Tensor<cpu, dim, float>
#define V1(p, len) View(p, Shape1(len))
#define V2(p, d0, d1) View(p, Shape2(d0, d1))
#define V2S(p, d0, d1, pitch) \
  Tensor<cpu, 2, float>(const_cast<float *>(p), Shape2(d0, d1), pitch, NULL)
#define V3(p, d0, d1, d2) View(p, Shape3(d0, d1, d2))
#include "../../mshadow_amd/cases/dot_cases.inc"
#undef XPU
#undef STREAM
#undef TENSOR
#undef V1
#undef V2
#undef V2S
#undef V3
  } catch (const std::exception &e) {
    fprintf(stderr, "%s\n", e.what());
    return 1;
  }
  return 0;
}

extern "C" int host_two_layer_net_f32(int steps, float eta, float decay, int batch, int n_in,
                                      int n_hidden, int n_out, const float *x, const float *label,
                                      float *w1, float *w2, float *probs) {
  try {
    two_layer_net::Train<cpu>(NULL, steps, eta, decay, View(x, Shape2(batch, n_in)),
                              View(label, Shape1(batch)), View(w1, Shape2(n_in, n_hidden)),
                              View(w2, Shape2(n_hidden, n_out)), View(probs, Shape2(batch, n_out)));
  } catch (const std::exception &e) {
    fprintf(stderr, "%s\n", e.what());
    return 1;
  }
  return 0;
}

static conv_net::Geometry GeometryOf(const int *v) {
  const conv_net::Geometry g = {v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8]};
  return g;
}

extern "C" int host_conv_net_f32(const int *geometry, int steps, float eta, float decay,
                                 const float *images, const float *labels, const float *fixed_grad,
                                 float *kernel, float *weight, float *const *keep) {
  try {
    conv_net::Train<cpu>(NULL, GeometryOf(geometry), steps, eta, decay, images, labels, fixed_grad,
                         kernel, weight, keep);
  } catch (const std::exception &e) {
    fprintf(stderr, "%s\n", e.what());
    return 1;
  }
  return 0;
}

extern "C" int host_conv_pair(int half, const int *geometry, const void *image, const void *kernel,
                              const void *grad_out, void *col_forward, void *out, void *col_backward,
                              void *image_grad) {
  typedef half::half_t H;
  try {
    if (half) {
      conv_net::ConvPair<cpu, H>(NULL, GeometryOf(geometry), static_cast<const H *>(image),
                                 static_cast<const H *>(kernel), static_cast<const H *>(grad_out),
                                 static_cast<H *>(col_forward), static_cast<H *>(out),
                                 static_cast<H *>(col_backward), static_cast<H *>(image_grad));
    } else {
      conv_net::ConvPair<cpu, float>(NULL, GeometryOf(geometry), static_cast<const float *>(image),
                                     static_cast<const float *>(kernel), static_cast<const float *>(grad_out),
                                     static_cast<float *>(col_forward), static_cast<float *>(out),
                                     static_cast<float *>(col_backward), static_cast<float *>(image_grad));
    }
  } catch (const std::exception &e) {
    fprintf(stderr, "%s\n", e.what());
    return 1;
  }
  return 0;
}
