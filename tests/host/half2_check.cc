// half2_t: arithmetic lane by lane in half_t, its DataType, the type switch that selects it, and
// an expression over a tensor of it - on Tensor<cpu> with any compiler, on Tensor<gpu> as well
// when the compiler is hipcc.
#include <mshadow/tensor.h>
using namespace mshadow; using namespace mshadow::expr;
typedef half::half2_t h2; typedef half::half_t h1;
int main() {
  static_assert(sizeof(h2) == 4 && alignof(h2) == 4, "two lanes");
  static_assert(DataType<h2>::kLanes == 2 && DataType<h2>::kFlag == kFloat16, "flag");
  h2 a(h1(1.5f), h1(-2.0f)), b(3);
  h2 c = a * b + a; c -= b; c /= h2(h1(2.0f), h1(4.0f));
  // (1.5*3+1.5-3)/2 = 1.5 ; (-2*3-2-3)/4 = -2.75
  int bad = !(float(c.half_t2[0]) == 1.5f && float(c.half_t2[1]) == -2.75f);
  bad += !((-a) == h2(h1(-1.5f), h1(2.0f)));
  bad += !((h2(h1(5.5f), h1(7.0f)) % h2(2)) == h2(h1(1.5f), h1(1.0f)));
  TensorContainer<cpu, 2, h2> x(Shape2(3, 4)), y(Shape2(3, 4));
  x = a; y = x * x + x;
  bad += !(y[2][3] == h2(h1(3.75f), h1(2.0f)));
  int lanes = 0;
  MSHADOW_TYPE_SWITCH_WITH_HALF2(kFloat16, DType, { lanes = DataType<DType>::kLanes; });
  bad += lanes != 2;
  int large_bytes = 0;
  MSHADOW_REAL_TYPE_SWITCH_EX(kFloat16, DType, DLarge, { large_bytes = sizeof(DType) * 10 + sizeof(DLarge); });
  bad += large_bytes != 24;
#if !MSHADOW_USE_CUDA || MSHADOW_USE_CUDNN || MSHADOW_USE_CBLAS
  bad += 1;  // the switches callers test: Tensor<gpu> exists, no cuDNN, no external host BLAS
#endif
#ifdef __HIPCC__
  Stream<gpu> *s = NewStream<gpu>();
  TensorContainer<gpu, 2, h2> gx(Shape2(3, 4)), gy(Shape2(3, 4));
  gx.set_stream(s); gy.set_stream(s);
  Copy(gx, x, s); gy = gx * gx + gx; Copy(x, gy, s); s->Wait();
  bad += !(x[2][3] == h2(h1(3.75f), h1(2.0f)));
  DeleteStream(s);
#endif
  printf(bad ? "BAD %d\n" : "OK\n", bad); return bad; }
