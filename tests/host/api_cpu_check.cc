// Host-only check of the mshadow C++ API of this repository (compiled with g++, no GPU):
// every hot-path expression is evaluated on Tensor<cpu> through the headers under
// mshadow_amd/mshadow/ and compared, bit for bit, with the C oracle (oracle/oracle.h).
// The Plan::Eval index math exercised here is the same code the generic GPU kernels run.
// Also checks API behaviour callers rely on: shapes, strides, CHECK failures that throw.
// Prints "OK <n> checks"; exit status 0 on success.
#define DMLC_LOG_FATAL_THROW 1
#include <mshadow/tensor.h>
#include <mshadow/io.h>

#include <cstdio>
#include <cstring>
#include <random>
#include <sstream>
#include <vector>

#include "../../mshadow_amd/cases/portable_math.h"
#include "../../oracle/oracle.h"

using namespace mshadow;
using namespace mshadow::expr;

struct sigmoid {
  MSHADOW_XINLINE static float Map(float a) { return pmath_sigmoid(a); }
};
struct maxoftwo {  // guide/defop.cpp:10-17 of the reference
  MSHADOW_XINLINE static float Map(float a, float b) { return a > b ? a : b; }
};

static int g_checks = 0, g_fail = 0;
#define EXPECT(cond)                                                        \
  do {                                                                      \
    ++g_checks;                                                             \
    if (!(cond)) {                                                          \
      ++g_fail;                                                             \
      fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);     \
    }                                                                       \
  } while (0)

template <typename T>
static bool SameBits(const T *a, const T *b, size_t n) { return memcmp(a, b, n * sizeof(T)) == 0; }

static std::vector<float> Rand(size_t n, unsigned seed, float lo = -1, float hi = 1) {
  std::mt19937 rng(seed);
  std::vector<float> v(n);
  for (auto &x : v) x = lo + (hi - lo) * (rng() >> 8) * (1.0f / 16777216.0f);
  return v;
}

template <typename Fn>
static bool Throws(Fn fn) {
  try {
    fn();
  } catch (const dmlc::Error &) {
    return true;
  }
  return false;
}

int main() {
  // ---- Shape / Tensor basics
  {
    Shape<4> s = Shape4(2, 3, 4, 5);
    EXPECT(s.Size() == 120 && s.FlatTo2D()[0] == 24 && s.FlatTo2D()[1] == 5);
    EXPECT(s.ProdShape(1, 3) == 12 && s.SubShape()[0] == 3);
    EXPECT((s.Slice<1, 3>()[1] == 4));
    std::ostringstream os;
    os << Shape2(2, 3) << Shape1(5);
    EXPECT(os.str() == "(2,3)(5,)");
    EXPECT(ConvertLayout(Shape4(1, 2, 3, 4), kNCHW, kNHWC) == Shape4(1, 3, 4, 2));
    EXPECT(ConvertLayout(Shape4(1, 3, 4, 2), kNHWC, kNCHW) == Shape4(1, 2, 3, 4));
    Tensor<cpu, 3> t = NewTensor<cpu>(Shape3(2, 3, 5), 1.5f);  // padded: 5 floats -> pitch 8
    EXPECT(t.stride_ == 8 && !t.CheckContiguous() && t.MSize() == 48);
    EXPECT(t[1][2][4] == 1.5f && t.Slice(1, 2).shape_[0] == 1);
    EXPECT(t[1].dptr_ == t.dptr_ + 3 * 8);
    FreeSpace(&t);
    Tensor<cpu, 2> u = NewTensor<cpu>(Shape2(3, 5), 0.0f, false);
    EXPECT(u.stride_ == 5 && u.CheckContiguous());
    FreeSpace(&u);
    TensorContainer<cpu, 2> c(Shape2(4, 6), 2.0f);
    c.Resize(Shape2(2, 3));
    EXPECT(c.size(0) == 2 && c.size(1) == 3);
    TensorContainer<cpu, 2> d(c);
    EXPECT(d[1][2] == 2.0f && d.dptr_ != c.dptr_);
    EXPECT(sizeof(half::half_t) == 2 && mshadow_sizeof(kFloat16) == 2 && DataType<float>::kFlag == 0);
  }
  // ---- elementwise map incl. savers, scalar rhs, user functors, padded tensors
  {
    const int R = 37, C = 129;
    std::vector<float> a = Rand(R * C, 1), b = Rand(R * C, 2), c = Rand(R * C, 3), d = Rand(R * C, 4);
    Tensor<cpu, 2> A(a.data(), Shape2(R, C)), B(b.data(), Shape2(R, C)), Cc(c.data(), Shape2(R, C)),
        D(d.data(), Shape2(R, C));
    for (int saver = 0; saver < 5; ++saver) {
      std::vector<float> o1 = Rand(R * C, 5, 1, 2), o2 = o1;
      Tensor<cpu, 2> O(o1.data(), Shape2(R, C));
      switch (saver) {
        case 0: O = A * B + 0.5f * F<sigmoid>(Cc) - D; break;
        case 1: O += A * B + 0.5f * F<sigmoid>(Cc) - D; break;
        case 2: O -= A * B + 0.5f * F<sigmoid>(Cc) - D; break;
        case 3: O *= A * B + 0.5f * F<sigmoid>(Cc) - D; break;
        default: O /= A * B + 0.5f * F<sigmoid>(Cc) - D; break;
      }
      orc_map_fused_f32(o2.data(), C, a.data(), C, b.data(), C, c.data(), C, d.data(), C, R, C, saver);
      EXPECT(SameBits(o1.data(), o2.data(), o1.size()));
    }
    TensorContainer<cpu, 2> P(Shape2(R, C)), Q(Shape2(R, C));  // padded rows
    Copy(P, A);
    Q = (P + 10.0f) / 3.0f + 2.0f;
    std::vector<float> want(R * C);
    orc_map_axpb_f32(want.data(), C, a.data(), C, R, C, 10.0f, 3.0f, 2.0f, 0);
    TensorContainer<cpu, 2> Qc(false);
    Qc.Resize(Shape2(R, C));
    Copy(Qc, Q);
    EXPECT(SameBits(Qc.dptr_, want.data(), want.size()));
    Q = F<maxoftwo>(P, 0.25f);
    EXPECT(Q[3][5] == (a[3 * C + 5] > 0.25f ? a[3 * C + 5] : 0.25f));
    Q = 3.0f;
    Q *= 2.0f;
    EXPECT(Q[R - 1][C - 1] == 6.0f);
    // transposed view and typecast
    TensorContainer<cpu, 2> Tt(Shape2(C, R));
    Tt = P.T();
    EXPECT(Tt[7][3] == P[3][7]);
    TensorContainer<cpu, 2, int32_t> I(Shape2(R, C));
    I = tcast<int32_t>(P * 10.0f);
    EXPECT(I[2][2] == static_cast<int32_t>(a[2 * C + 2] * 10.0f));
    // shape mismatch is a CHECK failure
    TensorContainer<cpu, 2> W(Shape2(R, C + 1));
    EXPECT(Throws([&] { Q = P + W; }));
  }
  // ---- reductions
  {
    const int N = 7, C = 5, Y = 9, X = 11;
    std::vector<float> x = Rand(N * C * Y * X, 6);
    Tensor<cpu, 4> T(x.data(), Shape4(N, C, Y, X));
    std::vector<float> o1(C, 1.0f), o2(C, 1.0f);
    Tensor<cpu, 1> O(o1.data(), Shape1(C));
    O += 0.5f * sumall_except_dim<1>(T);
    orc_reduce_keep_highdim_f32(o2.data(), x.data(), X, N, C, Y, X, ORC_SUM, ORC_PLUSTO, 0.5f);
    EXPECT(SameBits(o1.data(), o2.data(), C));
    O = reduce_except_dim<1, red::maximum>(T);
    orc_reduce_keep_highdim_f32(o2.data(), x.data(), X, N, C, Y, X, ORC_MAX, ORC_SAVETO, 1.0f);
    EXPECT(SameBits(o1.data(), o2.data(), C));
    Tensor<cpu, 2> M = T.FlatTo2D();
    std::vector<float> r1(X), r2(X);
    Tensor<cpu, 1> Rr(r1.data(), Shape1(X));
    Rr = sum_rows(M);
    orc_reduce_keep_lowest_f32(r2.data(), x.data(), X, N * C * Y, X, ORC_SUM, ORC_SAVETO, 1.0f);
    EXPECT(SameBits(r1.data(), r2.data(), X));
    Rr = sum_rows(M * 2.0f);  // an expression as the source (doc/README.md:162-168 form)
    std::vector<float> x2(x);
    for (auto &v : x2) v = v * 2.0f;
    orc_reduce_keep_lowest_f32(r2.data(), x2.data(), X, N * C * Y, X, ORC_SUM, ORC_SAVETO, 1.0f);
    EXPECT(SameBits(r1.data(), r2.data(), X));
    // keep dimension 0 of a 3-D tensor (test/test.cu:44-52 of the reference)
    std::vector<float> z1(N), z2(N);
    Tensor<cpu, 3> T3(x.data(), Shape3(N, C * Y, X));
    Tensor<cpu, 1> Z(z1.data(), Shape1(N));
    Z = sumall_except_dim<0>(T3);
    orc_reduce_keep_highdim_f32(z2.data(), x.data(), X, 1, N, C * Y, X, ORC_SUM, ORC_SAVETO, 1.0f);
    EXPECT(SameBits(z1.data(), z2.data(), N));
    Tensor<cpu, 1> Bad(z1.data(), Shape1(N + 1));
    EXPECT(Throws([&] { Bad = sumall_except_dim<0>(T3); }));
  }
  // ---- softmax and its gradient
  {
    const int R = 9, C = 1000;
    std::vector<float> x = Rand(R * C, 7, -9, 9), o1(R * C), o2(R * C), lab(R);
    for (int i = 0; i < R; ++i) lab[i] = static_cast<float>((i * 131) % C);
    lab[2] = -4.0f;
    lab[3] = C + 10.0f;
    Tensor<cpu, 2> X(x.data(), Shape2(R, C)), O(o1.data(), Shape2(R, C));
    Softmax(O, X);
    orc_softmax_f32(o2.data(), C, x.data(), C, R, C);
    EXPECT(SameBits(o1.data(), o2.data(), o1.size()));
    std::vector<float> g1(R * C), g2(R * C);
    Tensor<cpu, 2> G(g1.data(), Shape2(R, C));
    SoftmaxGrad(G, O, Tensor<cpu, 1>(lab.data(), Shape1(R)));
    orc_softmax_grad_f32(g2.data(), C, o2.data(), C, lab.data(), R, C);
    EXPECT(SameBits(g1.data(), g2.data(), g1.size()));
  }
  // ---- pool / unpool
  for (int reducer = 0; reducer < 3; ++reducer) {
    const int P = 4, H = 23, W = 17, ky = 3, kx = 2, sy = 2, sx = 3;
    const int PH = (H - ky) / sy + 1, PW = (W - kx) / sx + 1;
    std::vector<float> x = Rand(P * H * W, 8);
    for (auto &v : x) v = floorf(v * 4) / 4;  // duplicates
    std::vector<float> p1(P * PH * PW), p2(p1), gr = Rand(P * PH * PW, 9), u1(P * H * W), u2(u1);
    Tensor<cpu, 3> X(x.data(), Shape3(P, H, W)), Po(p1.data(), Shape3(P, PH, PW)),
        G(gr.data(), Shape3(P, PH, PW)), U(u1.data(), Shape3(P, H, W));
    if (reducer == 0) {
      Po = pool<red::sum>(X, ky, kx, sy, sx);
      U = unpool<red::sum>(X, Po, G, ky, kx, sy, sx);
    } else if (reducer == 1) {
      Po = pool<red::maximum>(X, ky, kx, sy, sx);
      U = unpool<red::maximum>(X, Po, G, ky, kx, sy, sx);
    } else {
      Po = pool<red::minimum>(X, ky, kx, sy, sx);
      U = unpool<red::minimum>(X, Po, G, ky, kx, sy, sx);
    }
    orc_pool_f32(p2.data(), PW, x.data(), W, P, H, W, PH, PW, ky, kx, sy, sx, reducer);
    orc_unpool_f32(u2.data(), W, x.data(), W, p2.data(), PW, gr.data(), PW, P, H, W, PH, PW, ky, kx,
                   sy, sx, reducer);
    EXPECT(SameBits(p1.data(), p2.data(), p1.size()));
    EXPECT(SameBits(u1.data(), u2.data(), u1.size()));
    EXPECT(Throws([&] { Po = pool<red::maximum>(X, H + 1, kx, sy, sx); }));
  }
  // ---- pad / crop / unpack_patch2col / pack_col2patch, float and half
  {
    const int N = 2, C = 3, H = 9, W = 8;
    struct Cfg { int ky, kx, sy, sx, dy, dx, py, px; };
    const Cfg cfgs[] = {{3, 3, 1, 1, 1, 1, 1, 1}, {3, 2, 2, 1, 1, 1, 0, 2}, {2, 3, 1, 2, 2, 2, 1, 0}};
    std::vector<float> img = Rand(N * C * H * W, 10);
    for (const Cfg &k : cfgs) {
      const int HP = H + 2 * k.py, WP = W + 2 * k.px;
      const int OH = (HP - (k.dy * (k.ky - 1) + 1)) / k.sy + 1, OW = (WP - (k.dx * (k.kx - 1) + 1)) / k.sx + 1;
      const int rows = k.ky * k.kx * C, cols = OH * OW * N;
      std::vector<float> c1(rows * cols), c2(c1), colin = Rand(rows * cols, 11), i1(img.size()), i2(i1);
      Tensor<cpu, 4> I(img.data(), Shape4(N, C, H, W)), I1(i1.data(), Shape4(N, C, H, W));
      Tensor<cpu, 2> Cm(c1.data(), Shape2(rows, cols)), Cin(colin.data(), Shape2(rows, cols));
      Cm = unpack_patch2col(pad(I, k.py, k.px), k.ky, k.kx, k.sy, k.sx, k.dy, k.dx);
      orc_im2col_f32(c2.data(), cols, img.data(), W, N, C, H, W, k.ky, k.kx, k.sy, k.sx, k.dy, k.dx, k.py, k.px);
      EXPECT(SameBits(c1.data(), c2.data(), c1.size()));
      I1 = crop(pack_col2patch(Cin, Shape4(N, C, HP, WP), k.ky, k.kx, k.sy, k.sx, k.dy, k.dx),
                Shape2(H, W), k.py, k.px);
      orc_col2im_f32(i2.data(), W, colin.data(), cols, N, C, H, W, k.ky, k.kx, k.sy, k.sx, k.dy, k.dx, k.py, k.px);
      EXPECT(SameBits(i1.data(), i2.data(), i1.size()));
      // half: values converted through half_t(float), accumulation rounds every step
      std::vector<half::half_t> hc(rows * cols), hi1(img.size());
      std::vector<uint16_t> hcb(rows * cols), hi2(img.size());
      bool half_encode_same = true;
      for (size_t i = 0; i < hc.size(); ++i) {
        hc[i] = half::half_t(colin[i] * 3.0f);
        hcb[i] = hc[i].half_;
        half_encode_same = half_encode_same && hcb[i] == orc_float2half(colin[i] * 3.0f);
      }
      EXPECT(half_encode_same);
      Tensor<cpu, 4, half::half_t> HI(hi1.data(), Shape4(N, C, H, W));
      Tensor<cpu, 2, half::half_t> HC(hc.data(), Shape2(rows, cols));
      HI = crop(pack_col2patch(HC, Shape4(N, C, HP, WP), k.ky, k.kx, k.sy, k.sx, k.dy, k.dx),
                Shape2(H, W), k.py, k.px);
      orc_col2im_f16(hi2.data(), W, hcb.data(), cols, N, C, H, W, k.ky, k.kx, k.sy, k.sx, k.dy, k.dx, k.py, k.px);
      EXPECT(memcmp(hi1.data(), hi2.data(), hi2.size() * 2) == 0);
    }
    Tensor<cpu, 4> I(img.data(), Shape4(N, C, H, W));
    TensorContainer<cpu, 4> padded(Shape4(N, C, H + 2, W + 4)), back(Shape4(N, C, H, W));
    padded = pad(I, 1, 2);
    EXPECT(padded[1][2][0][3] == 0.0f && padded[1][2][1][2] == I[1][2][0][0]);
    back = crop(padded, Shape2(H, W));  // centred crop undoes the symmetric pad
    EXPECT(back[1][1][4][5] == I[1][1][4][5] && back[0][0][0][0] == I[0][0][0][0]);
  }
  // ---- the rest of the softmax family and the row scatter / gather functions
  {
    const int R = 7, C = 13;
    std::vector<float> p = Rand(R * C, 20, 0, 1), lab = {0, 12, 4, 4, -2, 13, 5};
    Tensor<cpu, 2> P(p.data(), Shape2(R, C));
    Tensor<cpu, 1> L(lab.data(), Shape1(R));
    for (int flags = 1; flags < 4; ++flags) {
      std::vector<float> o1(R * C), o2(R * C);
      Tensor<cpu, 2> O(o1.data(), Shape2(R, C));
      if (flags == 1) SmoothSoftmaxGrad(O, P, L, 0.1f);
      else if (flags == 2) SoftmaxGrad(O, P, L, 4.0f);
      else SmoothSoftmaxGrad(O, P, L, 4.0f, 0.1f);
      orc_softmax_grad_ex_f32(o2.data(), C, p.data(), C, lab.data(), R, C, flags, 4.0f, 0.1f);
      EXPECT(SameBits(o1.data(), o2.data(), o1.size()));
    }
    const int D0 = 3, D1 = 6, D2 = 5;
    std::vector<float> x = Rand(D0 * D1 * D2, 21, -6, 6), s1(x.size()), s2(x.size());
    Tensor<cpu, 3> X(x.data(), Shape3(D0, D1, D2)), S(s1.data(), Shape3(D0, D1, D2));
    Softmax(S, X);
    orc_softmax3d_f32(s2.data(), D2, x.data(), D2, D0, D1, D2);
    EXPECT(SameBits(s1.data(), s2.data(), s1.size()));
    std::vector<float> l3 = Rand(D0 * D2, 22, 0, 5.99f);
    Tensor<cpu, 2> L3(l3.data(), Shape2(D0, D2));
    for (int flags = 0; flags < 4; ++flags) {
      std::vector<float> g1(x.size()), g2(x.size());
      Tensor<cpu, 3> Gt(g1.data(), Shape3(D0, D1, D2));
      if (flags == 0) SoftmaxGrad(Gt, S, L3);
      else if (flags == 1) SmoothSoftmaxGrad(Gt, S, L3, 0.2f);
      else if (flags == 2) SoftmaxGrad(Gt, S, L3, 3.0f);
      else SmoothSoftmaxGrad(Gt, S, L3, 3.0f, 0.2f);
      orc_softmax3d_grad_f32(g2.data(), D2, s2.data(), D2, l3.data(), D2, D0, D1, D2, flags, 3.0f, 0.2f);
      EXPECT(SameBits(g1.data(), g2.data(), g1.size()));
    }
    const int K = 5, N = 40, W = 3;
    std::vector<float> src = Rand(N * W, 23), d1 = Rand(K * W, 24), d2 = d1;
    std::vector<int> idx(N), srt(N), ord(N);
    for (int i = 0; i < N; ++i) idx[i] = (i * 7) % 9 - 2;
    Tensor<cpu, 2> Sr(src.data(), Shape2(N, W)), Dd(d1.data(), Shape2(K, W));
    Tensor<cpu, 1, int> I(idx.data(), Shape1(N));
    AddTakeGrad(Dd, I, Sr);
    orc_add_take_grad_f32(d2.data(), W, K, idx.data(), 1, N, src.data(), W, W);
    EXPECT(SameBits(d1.data(), d2.data(), d1.size()));
    for (int i = 0; i < N; ++i) { srt[i] = i * K / N; ord[i] = (i * 17) % N; }
    Tensor<cpu, 1, int> So(srt.data(), Shape1(N)), Or(ord.data(), Shape1(N));
    AddTakeGradLargeBatch(Dd, So, Or, Sr);
    orc_add_take_grad_large_batch_f32(d2.data(), W, srt.data(), ord.data(), 1, N, src.data(), W, W);
    EXPECT(SameBits(d1.data(), d2.data(), d1.size()));
    IndexFill(Dd, So, Sr);
    orc_index_fill_f32(d2.data(), W, srt.data(), 1, N, src.data(), W, W);
    EXPECT(SameBits(d1.data(), d2.data(), d1.size()));
  }
  // ---- SaveBinary / LoadBinary: the record is the shape followed by the dense rows
  {
    struct MemStream : public utils::IStream {
      std::vector<char> bytes;
      size_t pos = 0;
      size_t Read(void *ptr, size_t size) override {
        const size_t n = std::min(size, bytes.size() - pos);
        memcpy(ptr, bytes.data() + pos, n);
        pos += n;
        return n;
      }
      void Write(const void *ptr, size_t size) override {
        const char *c = static_cast<const char *>(ptr);
        bytes.insert(bytes.end(), c, c + size);
      }
    } ms;
    TensorContainer<cpu, 3> t(Shape3(2, 3, 5));   // padded rows: the pitch is not stored
    for (index_t i = 0; i < 2; ++i) for (index_t j = 0; j < 3; ++j) for (index_t k = 0; k < 5; ++k)
      t[i][j][k] = static_cast<float>(100 * i + 10 * j + k);
    SaveBinary(ms, t);
    EXPECT(ms.bytes.size() == 3 * sizeof(index_t) + 30 * sizeof(float));
    index_t stored[3];
    memcpy(stored, ms.bytes.data(), sizeof(stored));
    EXPECT(stored[0] == 2 && stored[1] == 3 && stored[2] == 5);
    float first_row[5];
    memcpy(first_row, ms.bytes.data() + sizeof(stored) + 5 * sizeof(float), sizeof(first_row));
    EXPECT(first_row[0] == 10.0f && first_row[4] == 14.0f);
    Tensor<cpu, 3> back;
    LoadBinary(ms, &back, false);
    bool same = back.shape_ == t.shape_;
    for (index_t i = 0; i < 2; ++i) for (index_t j = 0; j < 3; ++j) for (index_t k = 0; k < 5; ++k)
      same = same && back[i][j][k] == t[i][j][k];
    EXPECT(same);
    FreeSpace(&back);
    ms.pos = 0;
    TensorContainer<cpu, 3> wrong(Shape3(2, 3, 4));
    EXPECT(Throws([&] { LoadBinary(ms, &wrong, true); }));
    // the container's own members: the same record, and LoadBinary takes the stored shape
    decltype(ms) cs;
    t.SaveBinary(cs);
    EXPECT(cs.bytes == ms.bytes);
    TensorContainer<cpu, 3> other(Shape3(1, 1, 2), 7.0f);
    other.LoadBinary(cs);
    same = other.shape_ == t.shape_;
    for (index_t i = 0; i < 2; ++i) for (index_t j = 0; j < 3; ++j) for (index_t k = 0; k < 5; ++k)
      same = same && other[i][j][k] == t[i][j][k];
    EXPECT(same);
    TensorContainer<cpu, 3> dense(false);   // into an empty, unpadded container
    cs.pos = 0;
    dense.LoadBinary(cs);
    EXPECT(dense.shape_ == t.shape_ && dense.stride_ == 5 && dense[1][2][4] == 124.0f);
  }
  // ---- TensorContainer: the view moves inside the block, a larger shape takes a new block
  {
    TensorContainer<cpu, 2> c(Shape2(8, 10), 1.0f);
    float *block = c.dptr_;
    const index_t pitch = c.stride_;
    EXPECT(pitch >= 10);
    c.Resize(Shape2(3, 7));                       // fits: same memory, padded pitch kept
    EXPECT(c.dptr_ == block && c.stride_ == pitch && c.size(0) == 3 && c.size(1) == 7);
    c.Resize(Shape2(8, 10));
    EXPECT(c.dptr_ == block);
    c.Resize(Shape2(9, 10), 4.0f);                // one row too many: a new block, filled
    EXPECT(c.size(0) == 9 && c[8][9] == 4.0f);
    TensorContainer<cpu, 2> d(false);
    EXPECT(d.dptr_ == NULL && d.shape_[0] == 0);
    d.Resize(Shape2(4, 6), 2.0f);
    EXPECT(d.stride_ == 6);
    d.Resize(Shape2(4, 3));                       // dense rows follow the shape
    EXPECT(d.stride_ == 3);
    TensorContainer<cpu, 2> e(c);                 // copies the elements
    EXPECT(e.dptr_ != c.dptr_ && e[8][9] == 4.0f);
    e = 5.0f;
    d = e;                                        // takes shape, padding choice and elements
    EXPECT(d.shape_ == e.shape_ && d[0][0] == 5.0f && c[0][0] == 4.0f);
    d.Release();
    EXPECT(d.dptr_ == NULL && d.shape_[0] == 0);
    d.Release();
  }
  // ---- SortByKey / VectorizedSort on the CPU device against the oracle
  {
    const int N = 777;
    std::vector<float> kf(N), kf2;
    std::vector<int> vi(N), vi2, seg(N), seg2;
    for (int i = 0; i < N; ++i) {
      kf[i] = static_cast<float>((i * 37) % 11 - 5) * 0.5f;
      if (i % 13 == 0) kf[i] = -0.0f;
      vi[i] = i;
      seg[i] = i / 50;
    }
    for (int ascend = 0; ascend < 2; ++ascend) {
      kf2 = kf; vi2 = vi;
      std::vector<float> a = kf; std::vector<int> b = vi;
      SortByKey(Tensor<cpu, 1, float>(a.data(), Shape1(N)), Tensor<cpu, 1, int>(b.data(), Shape1(N)),
                ascend != 0);
      orc_sort_by_key_32(kf2.data(), 0, vi2.data(), N, ascend);
      EXPECT(SameBits(a.data(), kf2.data(), N) && b == vi2);
    }
    kf2 = kf; seg2 = seg;
    std::vector<float> a = kf;
    VectorizedSort(Tensor<cpu, 1, float>(a.data(), Shape1(N)), Tensor<cpu, 1, int>(seg.data(), Shape1(N)));
    orc_vectorized_sort_32(kf2.data(), 0, seg2.data(), N);
    EXPECT(SameBits(a.data(), kf2.data(), N) && seg == seg2);
  }
  // ---- index-remapping extensions on the CPU device, against plain index loops
  {
    const int n = 2, c = 3, h = 4, w = 5;
    std::vector<float> a = Rand(n * c * h * w, 30), v = Rand(n * c * h * w, 31);
    auto A = [&](int i, int j, int k, int l) { return a[((i * c + j) * h + k) * w + l]; };
    Tensor<cpu, 4> In(a.data(), Shape4(n, c, h, w));
    Tensor<cpu, 1> Vc(v.data(), Shape1(c)), Vw(v.data(), Shape1(w));
    TensorContainer<cpu, 4> o(Shape4(n, c, h, w));
    o = In + broadcast<1>(Vc, o.shape_);
    bool ok = true;
    for (int i = 0; i < n; ++i) for (int j = 0; j < c; ++j) for (int k = 0; k < h; ++k)
      for (int l = 0; l < w; ++l) ok = ok && o[i][j][k][l] == A(i, j, k, l) + v[j];
    EXPECT(ok);
    TensorContainer<cpu, 2> o2(Shape2(n * c * h, w));
    o2 = In.FlatTo2D() + repmat(Vw, n * c * h);
    ok = true;
    for (int r = 0; r < n * c * h; ++r) for (int l = 0; l < w; ++l) ok = ok && o2[r][l] == a[r * w + l] + v[l];
    EXPECT(ok);
    TensorContainer<cpu, 4> sw(Shape4(c, n, h, w));
    sw = swapaxis<1, 0>(reshape(Tensor<cpu, 2>(a.data(), Shape2(n, c * h * w)), Shape4(n, c, h, w)));
    ok = true;
    for (int i = 0; i < n; ++i) for (int j = 0; j < c; ++j) for (int k = 0; k < h; ++k)
      for (int l = 0; l < w; ++l) ok = ok && sw[j][i][k][l] == A(i, j, k, l);
    EXPECT(ok);
    TensorContainer<cpu, 4> s31(Shape4(n, w, h, c)), s21(Shape4(n, h, c, w)), mi(Shape4(n, c, h, w)),
        up(Shape4(n, c, 2 * h, 2 * w));
    s31 = swapaxis<3, 1>(In);
    s21 = swapaxis<2, 1>(In);
    mi = mirror(In);
    up = upsampling_nearest(In, 2);
    ok = true;
    for (int i = 0; i < n; ++i) for (int j = 0; j < c; ++j) for (int k = 0; k < h; ++k)
      for (int l = 0; l < w; ++l) {
        ok = ok && s31[i][l][k][j] == A(i, j, k, l) && s21[i][k][j][l] == A(i, j, k, l) &&
             mi[i][j][k][w - 1 - l] == A(i, j, k, l) && up[i][j][2 * k + 1][2 * l] == A(i, j, k, l) &&
             up[i][j][2 * k][2 * l + 1] == A(i, j, k, l);
      }
    EXPECT(ok);
    // guide/basic.cpp:127-134 of the reference: sum-pooling an upsampled tensor gives 9 x the source
    TensorContainer<cpu, 4> pooled(Shape4(n, c, h, w)), up3(Shape4(n, c, 3 * h, 3 * w));
    up3 = upsampling_nearest(In, 3);
    pooled = pool<red::sum>(up3, 3, 3, 3, 3);
    EXPECT(std::fabs(pooled[1][2][3][4] - 9.0f * A(1, 2, 3, 4)) < 1e-5f);
    Tensor<cpu, 1> one(v.data(), Shape1(1));
    o = broadcast_scalar(one, o.shape_) * In;
    EXPECT(o[1][1][1][1] == v[0] * A(1, 1, 1, 1));
    EXPECT(Throws([&] { o = In + broadcast<1>(Vw, o.shape_); }));          // length != shape[1]
    EXPECT(Throws([&] { o2 = reshape(In, Shape2(n * c * h, w + 1)); }));    // size mismatch
  }
  if (g_fail) {
    fprintf(stderr, "%d of %d checks failed\n", g_fail, g_checks);
    return 1;
  }
  printf("OK %d checks\n", g_checks);
  return 0;
}
