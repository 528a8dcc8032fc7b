// A caller that is compiled by the host compiler only (no device compiler) can still use
// everything of Tensor<gpu> that sits behind the C ABI: allocation, copies, streams and the
// assignments that are recognised as fixed-function operations. This file is compiled and
// linked by the CPU test suite (it proves the claim at build time) and run by a GPU test.
#include <mshadow/tensor.h>
#include <mshadow/io.h>
#include <mshadow/random.h>

#include <cstdio>
#include <cstring>
#include <vector>

using namespace mshadow;
using namespace mshadow::expr;

// An operator templated over its element type may hold a generator it never samples from:
// the class instantiates for every DType (sampling anything but float and double does not
// compile, as with the reference's float* / double* generator calls).
template <typename DType>
struct HoldsAGenerator {
  Random<gpu, DType> *rnd;
  size_t Footprint() const { return sizeof(Random<gpu, DType>); }
};
template struct HoldsAGenerator<half::half_t>;
template struct HoldsAGenerator<int>;

// The map kernels count in 32 bits; a larger view is evaluated in runs of whole rows. Nothing
// in that split may narrow: for any row length the run stays below 2^31 units with room for
// the last workgroup's reach, and covers at least one row.
static bool RunsOfRowsFit() {
  const uint32_t lengths[] = {1u, 3u, 4096u, 32768u, 65535u, (1u << 30) + 5u, 0x7fffffffu};
  for (uint32_t units : lengths) {
    const uint64_t rows = gpu_detail::RowsPerLaunch(units);
    if (rows < 1) return false;
    if (rows > 1 && rows * units + (1u << 16) > (1ull << 31)) return false;
    if ((rows + 1) * units + (1u << 16) <= (1ull << 31) && rows != 0xffffffffull) return false;  // not the largest run
  }
  return true;
}

int main() {
  if (!RunsOfRowsFit()) {
    std::printf("FAIL runs of rows\n");
    return 1;
  }
  InitTensorEngine<gpu>(0);
  Stream<gpu> *s = NewStream<gpu>(0);
  const int n = 2, c = 3, h = 9, w = 12;
  std::vector<float> host(n * c * h * w);
  for (size_t i = 0; i < host.size(); ++i) host[i] = static_cast<float>((i * 37) % 101) - 50.0f;
  Tensor<cpu, 4> hx(host.data(), Shape4(n, c, h, w));
  Tensor<gpu, 4> x = NewTensor<gpu>(Shape4(n, c, h, w), 0.0f, false, s);
  Tensor<gpu, 4> p = NewTensor<gpu>(Shape4(n, c, 4, 5), 0.0f, false, s);
  Tensor<gpu, 4> g = NewTensor<gpu>(Shape4(n, c, h, w), 0.0f, false, s);
  Tensor<gpu, 4> t = NewTensor<gpu>(Shape4(n, h, w, c), 0.0f, false, s);
  Tensor<gpu, 2> m = NewTensor<gpu>(Shape2(n * c * h, w), 0.0f, false, s);
  Tensor<gpu, 1> v = NewTensor<gpu>(Shape1(w), 0.0f, false, s);
  Copy(x, hx, s);
  p = pool<red::maximum>(x, 3, 3, 2, 2);
  g = unpool<red::maximum>(x, p, p, 3, 3, 2, 2);
  t = transpose(x, Shape4(0, 2, 3, 1));
  Copy(m, x.FlatTo2D(), s);
  v = sum_rows(m);
  Softmax(m, m);
  // expected values on the host with the CPU device of the same headers
  TensorContainer<cpu, 4> cp(Shape4(n, c, 4, 5)), ct(Shape4(n, h, w, c));
  TensorContainer<cpu, 1> cv(Shape1(w));
  cp = pool<red::maximum>(hx, 3, 3, 2, 2);
  ct = transpose(hx, Shape4(0, 2, 3, 1));
  cv = sum_rows(hx.FlatTo2D());
  TensorContainer<cpu, 4> gp(Shape4(n, c, 4, 5)), gt(Shape4(n, h, w, c));
  TensorContainer<cpu, 1> gv(Shape1(w));
  Copy(gp, p, s);
  Copy(gt, t, s);
  Copy(gv, v, s);
  s->Wait();
  int bad_pool = 0, bad_transpose = 0, bad_sum = 0;
  /* the containers pad their rows: compare element by element, not the raw buffers */
  Tensor<cpu, 2> cp2 = cp.FlatTo2D(), gp2 = gp.FlatTo2D(), ct2 = ct.FlatTo2D(), gt2 = gt.FlatTo2D();
  for (index_t y = 0; y < cp2.size(0); ++y)
    for (index_t x = 0; x < cp2.size(1); ++x) bad_pool += cp2[y][x] != gp2[y][x];
  for (index_t y = 0; y < ct2.size(0); ++y)
    for (index_t x = 0; x < ct2.size(1); ++x) bad_transpose += ct2[y][x] != gt2[y][x];
  for (index_t i = 0; i < cv.size(0); ++i) bad_sum += cv[i] != gv[i];
  int bad = 0;
  /* a device tensor written to a byte stream and read back into a new device tensor */
  struct MemStream {
    std::vector<char> bytes;
    size_t pos = 0;
    size_t Read(void *ptr, size_t size) {
      const size_t k = size < bytes.size() - pos ? size : bytes.size() - pos;
      memcpy(ptr, bytes.data() + pos, k);
      pos += k;
      return k;
    }
    void Write(const void *ptr, size_t size) {
      const char *c = static_cast<const char *>(ptr);
      bytes.insert(bytes.end(), c, c + size);
    }
  } ms;
  SaveBinary(ms, t);
  Tensor<gpu, 4> t2;
  t2.set_stream(s);
  LoadBinary(ms, &t2, false);
  TensorContainer<cpu, 4> gt_again(Shape4(n, h, w, c));
  Copy(gt_again, t2, s);
  s->Wait();
  Tensor<cpu, 2> again2 = gt_again.FlatTo2D();
  for (index_t y = 0; y < ct2.size(0); ++y)
    for (index_t x2 = 0; x2 < ct2.size(1); ++x2) bad_transpose += ct2[y][x2] != again2[y][x2];
  FreeSpace(&t2);
  /* the members of a device container: the same record; LoadBinary takes the stored shape */
  {
    decltype(ms) cs;
    TensorContainer<gpu, 4> dev(t.shape_), dev2(Shape4(1, 1, 1, 2));
    dev.set_stream(s), dev2.set_stream(s);
    Copy(dev, t, s);
    dev.SaveBinary(cs);
    bad_transpose += cs.bytes != ms.bytes;
    dev2.LoadBinary(cs);
    bad_transpose += !(dev2.shape_ == t.shape_);
    Copy(gt_again, dev2, s);
    s->Wait();
    for (index_t y = 0; y < ct2.size(0); ++y)
      for (index_t x2 = 0; x2 < ct2.size(1); ++x2) bad_transpose += ct2[y][x2] != again2[y][x2];
  }
  /* matrix products are library calls behind the ABI: (3x5 of i+j) x (4x5 of i-j)^T, and the
     scalar product of two of the rows, in small integers (exact in float) */
  int bad_dot = 0;
  {
    TensorContainer<cpu, 2> ha(Shape2(3, 5)), hb(Shape2(4, 5)), hc(Shape2(3, 4));
    TensorContainer<cpu, 1> hd(Shape1(1));
    for (index_t i = 0; i < 3; ++i) for (index_t j = 0; j < 5; ++j) ha[i][j] = static_cast<float>(i + j);
    for (index_t i = 0; i < 4; ++i) for (index_t j = 0; j < 5; ++j) hb[i][j] = static_cast<float>(i) - j;
    TensorContainer<gpu, 2> da(ha.shape_), db(hb.shape_), dc(hc.shape_);
    TensorContainer<gpu, 1> dd(Shape1(1));
    da.set_stream(s), db.set_stream(s), dc.set_stream(s), dd.set_stream(s);
    Copy(da, ha, s);
    Copy(db, hb, s);
    dc = 1.0f;
    dc += 2.0f * dot(da, db.T());
    VectorDot(dd, da[2], db[3]);
    Copy(hc, dc, s);
    Copy(hd, dd, s);
    s->Wait();
    float vd = 0.0f;
    for (index_t j = 0; j < 5; ++j) vd += ha[2][j] * hb[3][j];
    bad_dot += hd[0] != vd;
    for (index_t i = 0; i < 3; ++i) {
      for (index_t k = 0; k < 4; ++k) {
        float want = 0.0f;
        for (index_t j = 0; j < 5; ++j) want += ha[i][j] * hb[k][j];
        bad_dot += hc[i][k] != 1.0f + 2.0f * want;
      }
    }
  }
  FreeSpace(&x); FreeSpace(&p); FreeSpace(&g); FreeSpace(&t); FreeSpace(&m); FreeSpace(&v);
  bad = bad_pool + bad_transpose + bad_sum + bad_dot;
  DeleteStream(s);
  ShutdownTensorEngine<gpu>();
  if (bad) {
    printf("values that differ: pool %d, transpose %d, sum_rows %d, dot %d\n", bad_pool, bad_transpose,
           bad_sum, bad_dot);
    return 1;
  }
  printf("OK\n");
  return 0;
}
