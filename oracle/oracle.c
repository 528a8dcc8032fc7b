/*
 * TEST INFRASTRUCTURE - not part of the shipped library. See oracle.h.
 *
 * Build: gcc -std=c99 -O2 -fopenmp -ffp-contract=off -fPIC -shared oracle.c -lm
 * (-ffp-contract=off matters: the reference never fuses a*b+c, and bit-exact
 * parity of the elementwise map depends on it.)
 *
 * Parity pins (what fixes each function besides reading the reference):
 *   map            brute-force parenthesised scalar loop; guide/basic.cpp:25-30 values
 *   reductions     test/test.cu:9-18,35,47 closed forms; doc/README.md:162-185; all-ones counts
 *   softmax        uniform logits -> 1/n exactly; shift invariance; float64 brute force.
 *                  Absolute values depend on libm expf: parity unpinned at the ulp level
 *                  (the reference's tests only compare CPU with GPU at 1e-4).
 *   softmax grad   -1 at the label column, identical copy elsewhere
 *   pool / unpool  test/pool.cu:29-48, test/pairtest.cu:29-77 closed forms
 *   patch2col      test/unpack.cu:29-59 closed form; index-valued images
 *   col2patch      coverage counts 4/6/9; adjoint identity with patch2col
 *   half           exhaustive round trip; F16C agreement where the host has it
 *   *_f16          (map a*b+c, reductions, pool, softmax pair on half_t) what 16-bit rounding
 *                  after every operation fixes: a sum of ones stops at 2048; 2048+1+1 = 2048
 *                  but 1+1+2048 = 2050; two inner sums of 3000 ones merge to 4096; n equal
 *                  logits give 1/min(n, 2048); (1+2^-10)^2 rounds to 1+2^-9 before the sum.
 *                  The softmax's exponentials again come from libm expf (unpinned at the
 *                  ulp level, though a 16-bit result rarely shows a last-bit difference)
 * and, where /root/reference is present, bit-for-bit agreement with the reference's
 * own headers compiled into oracle/_ref (see oracle/Makefile).
 */
#include "oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#include "../mshadow_amd/cases/portable_math.h"

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------ half */

/* mshadow/half.h:197-242 (software path) and :321-330 (F16C, rounding mode 0):
   round to nearest, ties to even; overflow to infinity; gradual underflow. */
uint16_t orc_float2half(float v) {
  uint32_t x;
  memcpy(&x, &v, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t a = x & 0x7fffffffu;
  if (a > 0x7f800000u) { /* NaN: quiet, keep the top payload bits */
    return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x1ffu));
  }
  if (a >= 0x38800000u) { /* normal half range or above */
    uint32_t r = a + 0xfffu + ((a >> 13) & 1u);
    uint32_t h = (r - 0x38000000u) >> 13;
    if (h >= 0x7c00u) h = 0x7c00u;
    return (uint16_t)(sign | h);
  }
  /* result is a half subnormal (unit 2^-24) or zero */
  uint32_t e = a >> 23;
  if (e < 102u) return (uint16_t)sign; /* below 2^-25: rounds to zero */
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  uint32_t shift = 126u - e; /* 14..24 */
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1u);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  return (uint16_t)(sign | q);
}

/* mshadow/half.h:244-283: exact widening */
float orc_half2float(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  uint32_t x;
  if (e == 0) {
    if (m == 0) {
      x = sign;
    } else {
      float f = (float)m * 5.9604644775390625e-08f; /* m * 2^-24, exact */
      memcpy(&x, &f, 4);
      x |= sign;
    }
  } else if (e == 31) {
    /* inf, or NaN with the payload kept and the quiet bit set: what the F16C conversion
       the reference is built with returns for a signalling NaN (mshadow/half.h:285-296) */
    x = sign | 0x7f800000u | (m << 13) | (m ? 0x00400000u : 0u);
  } else {
    x = sign | ((e + 112u) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &x, 4);
  return f;
}

void orc_float2half_n(uint16_t *dst, const float *src, int64_t n) {
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) dst[i] = orc_float2half(src[i]);
}

void orc_half2float_n(float *dst, const uint16_t *src, int64_t n) {
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) dst[i] = orc_half2float(src[i]);
}

/* half_t arithmetic: every operator widens, computes in float and rounds back
   (mshadow/half.h:45-66); operator+= rounds after each step (:58-62) */
static inline uint16_t half_add(uint16_t a, uint16_t b) {
  return orc_float2half(orc_half2float(a) + orc_half2float(b));
}

/* ------------------------------------------------------------------ savers / reducers */

/* mshadow/base.h:539-602 */
static inline void save_f32(float *dst, float v, int saver) {
  switch (saver) {
    case ORC_SAVETO: *dst = v; break;
    case ORC_PLUSTO: *dst += v; break;
    case ORC_MINUSTO: *dst -= v; break;
    case ORC_MULTO: *dst *= v; break;
    default: *dst /= v; break;
  }
}

/* mshadow/base.h:676-680 (sum), :752-761 (maximum = std::max(dst, src)),
   :822-831 (minimum = std::min(dst, src)) */
static inline void reduce_f32(float *dst, float src, int reducer) {
  switch (reducer) {
    case ORC_SUM: *dst += src; break;
    case ORC_MAX: *dst = (*dst < src) ? src : *dst; break;
    default: *dst = (src < *dst) ? src : *dst; break;
  }
}

/* mshadow/base.h:716-719, :794-797, :858-861 */
static inline float init_f32(int reducer) {
  switch (reducer) {
    case ORC_SUM: return 0.0f;
    case ORC_MAX: return -FLT_MAX;
    default: return FLT_MAX;
  }
}

/* mshadow/base.h:711-714 (sum: 1), :787-790 and :851-854 (equality) */
static inline float partial_grad_f32(float redres, float redsrc, int reducer) {
  if (reducer == ORC_SUM) return 1.0f;
  return redres == redsrc ? 1.0f : 0.0f;
}

/* ------------------------------------------------------------------ elementwise map */

/* MapPlan, mshadow/tensor_cpu-inl.h:143-159: one thread per row y, x ascending,
   Saver::Save(dst(y,x), plan.Eval(y,x)). The expression tree
   A*B + 0.5f*F<sigmoid>(C) - D evaluates as ((a*b) + (0.5f*sig(c))) - d
   (mshadow/expression.h:353-374, expr_engine-inl.h:116-131). */
void orc_map_fused_f32(float *dst, int dstride, const float *a, int astride, const float *b,
                       int bstride, const float *c, int cstride, const float *d, int dstride_d,
                       int rows, int cols, int saver) {
#pragma omp parallel for
  for (int y = 0; y < rows; ++y) {
    for (int x = 0; x < cols; ++x) {
      float ab = a[(int64_t)y * astride + x] * b[(int64_t)y * bstride + x];
      float hs = 0.5f * pmath_sigmoid(c[(int64_t)y * cstride + x]);
      float v = (ab + hs) - d[(int64_t)y * dstride_d + x];
      save_f32(&dst[(int64_t)y * dstride + x], v, saver);
    }
  }
}

/* scalar right-hand side: Plan<ScalarExp>, mshadow/expr_engine-inl.h:83-93 */
void orc_map_scalar_f32(float *dst, int dstride, int rows, int cols, float scalar, int saver) {
#pragma omp parallel for
  for (int y = 0; y < rows; ++y) {
    for (int x = 0; x < cols; ++x) save_f32(&dst[(int64_t)y * dstride + x], scalar, saver);
  }
}

/* ((a + s1) / s2) + s3, the expression of guide/basic.cpp:27 */
void orc_map_axpb_f32(float *dst, int dstride, const float *a, int astride, int rows, int cols,
                      float s1, float s2, float s3, int saver) {
#pragma omp parallel for
  for (int y = 0; y < rows; ++y) {
    for (int x = 0; x < cols; ++x) {
      float v = ((a[(int64_t)y * astride + x] + s1) / s2) + s3;
      save_f32(&dst[(int64_t)y * dstride + x], v, saver);
    }
  }
}

/* ------------------------------------------------------------------ reductions */

/* MapReduceKeepLowest, mshadow/tensor_cpu-inl.h:203-228: one thread per column,
   res = src(0,x), then rows 1.. in order, Save(dst[x], res * scale). */
void orc_reduce_keep_lowest_f32(float *dst, const float *src, int sstride, int rows, int cols,
                                int reducer, int saver, float scale) {
#pragma omp parallel for
  for (int x = 0; x < cols; ++x) {
    float res = src[x];
    for (int y = 1; y < rows; ++y) reduce_f32(&res, src[(int64_t)y * sstride + x], reducer);
    save_f32(&dst[x], res * scale, saver);
  }
}

/* MapReduceKeepHighDim, mshadow/tensor_cpu-inl.h:230-268: shape viewed as
   (n, c, y, x); per kept index c: for each n an inner reduction over (y, x) from the
   reducer's initial value, merged in n order into the outer accumulator. */
void orc_reduce_keep_highdim_f32(float *dst, const float *src, int sstride, int n, int c, int y,
                                 int x, int reducer, int saver, float scale) {
#pragma omp parallel for
  for (int ci = 0; ci < c; ++ci) {
    float res = init_f32(reducer);
    for (int ni = 0; ni < n; ++ni) {
      float tres = init_f32(reducer);
      for (int yi = 0; yi < y; ++yi) {
        const float *row = src + (int64_t)((ni * c + ci) * y + yi) * sstride;
        for (int xi = 0; xi < x; ++xi) reduce_f32(&tres, row[xi], reducer);
      }
      reduce_f32(&res, tres, reducer);
    }
    save_f32(&dst[ci], res * scale, saver);
  }
}

/* ------------------------------------------------------------------ softmax */

/* Softmax, mshadow/tensor_cpu-inl.h:270-285 (one row) and :464-472 (rows in
   parallel): max with a strict '<' update, exp(x - max) written to dst and summed
   left to right in float, then a true division per element. In-place is allowed
   because each element of the row is read before it is written. */
void orc_softmax_f32(float *dst, int dstride, const float *src, int sstride, int rows, int cols) {
#pragma omp parallel for
  for (int y = 0; y < rows; ++y) {
    const float *e = src + (int64_t)y * sstride;
    float *o = dst + (int64_t)y * dstride;
    float mmax = e[0];
    for (int x = 1; x < cols; ++x) {
      if (mmax < e[x]) mmax = e[x];
    }
    float sum = 0.0f;
    for (int x = 0; x < cols; ++x) {
      o[x] = expf(e[x] - mmax);
      sum += o[x];
    }
    for (int x = 0; x < cols; ++x) o[x] /= sum;
  }
}

/* SoftmaxGrad, mshadow/tensor_cpu-inl.h:287-302: label is stored in the data
   type and truncated with static_cast<int>; a label outside [0, cols) leaves a copy. */
void orc_softmax_grad_f32(float *dst, int dstride, const float *src, int sstride,
                          const float *label, int rows, int cols) {
#pragma omp parallel for
  for (int y = 0; y < rows; ++y) {
    const int k = (int)label[y];
    const float *s = src + (int64_t)y * sstride;
    float *o = dst + (int64_t)y * dstride;
    for (int x = 0; x < cols; ++x) {
      if (x == k) {
        o[k] = s[k] - 1.0f;
      } else {
        o[x] = s[x];
      }
    }
  }
}

/* ---- the same functions on half_t tensors (16-bit storage). Every half_t operator widens
   to float, computes, and rounds back to 16 bits (mshadow/half.h:45-66), so each step of
   an accumulation rounds: a sum of ones stops growing at 2048. Comparisons are made on the
   widened values (:341-348). */
static inline uint16_t half_of(float v) { return orc_float2half(v); }
static inline float wide(uint16_t h) { return orc_half2float(h); }

static inline void save_f16(uint16_t *dst, uint16_t v, int saver) {
  switch (saver) {
    case ORC_SAVETO: *dst = v; break;
    case ORC_PLUSTO: *dst = half_of(wide(*dst) + wide(v)); break;
    case ORC_MINUSTO: *dst = half_of(wide(*dst) - wide(v)); break;
    case ORC_MULTO: *dst = half_of(wide(*dst) * wide(v)); break;
    default: *dst = half_of(wide(*dst) / wide(v)); break;
  }
}

/* red::sum / maximum / minimum on half_t (mshadow/base.h:692-697, :751-761, :807-817:
   std::max(dst, src) returns src only when dst < src, std::min only when src < dst) */
static inline void reduce_f16(uint16_t *dst, uint16_t src, int reducer) {
  switch (reducer) {
    case ORC_SUM: *dst = half_add(*dst, src); break;
    case ORC_MAX: *dst = (wide(*dst) < wide(src)) ? src : *dst; break;
    default: *dst = (wide(src) < wide(*dst)) ? src : *dst; break;
  }
}

/* mshadow/base.h:716-719 (0), :798-801 (MSHADOW_HALF_MIN = 0xFBFF), :862-865
   (MSHADOW_HALF_MAX = 0x7BFF) */
static inline uint16_t init_f16(int reducer) {
  switch (reducer) {
    case ORC_SUM: return 0;
    case ORC_MAX: return 0xFBFFu;
    default: return 0x7BFFu;
  }
}

/* dst <saver>= a * b + c on half_t tensors: the product is a half_t (rounded) before the
   sum is taken (mshadow/half.h:45-66, expression.h:353-374) */
void orc_map_muladd_f16(uint16_t *dst, int dstride, const uint16_t *a, int astride,
                        const uint16_t *b, int bstride, const uint16_t *c, int cstride, int rows,
                        int cols, int saver) {
#pragma omp parallel for
  for (int y = 0; y < rows; ++y) {
    for (int x = 0; x < cols; ++x) {
      const uint16_t ab = half_of(wide(a[(int64_t)y * astride + x]) * wide(b[(int64_t)y * bstride + x]));
      const uint16_t v = half_of(wide(ab) + wide(c[(int64_t)y * cstride + x]));
      save_f16(&dst[(int64_t)y * dstride + x], v, saver);
    }
  }
}

/* MapReduceKeepLowest on half_t, mshadow/tensor_cpu-inl.h:203-228 */
void orc_reduce_keep_lowest_f16(uint16_t *dst, const uint16_t *src, int sstride, int rows,
                                int cols, int reducer, int saver, uint16_t scale) {
#pragma omp parallel for
  for (int x = 0; x < cols; ++x) {
    uint16_t res = src[x];
    for (int y = 1; y < rows; ++y) reduce_f16(&res, src[(int64_t)y * sstride + x], reducer);
    save_f16(&dst[x], half_of(wide(res) * wide(scale)), saver);
  }
}

/* MapReduceKeepHighDim on half_t, mshadow/tensor_cpu-inl.h:230-268 */
void orc_reduce_keep_highdim_f16(uint16_t *dst, const uint16_t *src, int sstride, int n, int c,
                                 int y, int x, int reducer, int saver, uint16_t scale) {
#pragma omp parallel for
  for (int ci = 0; ci < c; ++ci) {
    uint16_t res = init_f16(reducer);
    for (int ni = 0; ni < n; ++ni) {
      uint16_t tres = init_f16(reducer);
      for (int yi = 0; yi < y; ++yi) {
        const uint16_t *row = src + (int64_t)((ni * c + ci) * y + yi) * sstride;
        for (int xi = 0; xi < x; ++xi) reduce_f16(&tres, row[xi], reducer);
      }
      reduce_f16(&res, tres, reducer);
    }
    save_f16(&dst[ci], half_of(wide(res) * wide(scale)), saver);
  }
}

/* Softmax on half_t, mshadow/tensor_cpu-inl.h:270-285: energy[x] - mmax is a half_t
   (rounded), std::exp takes it as a float and its result is rounded into dst[x]; the sum
   is a half_t that rounds after every add; dst[x] /= sum is a float division rounded. */
void orc_softmax_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride, int rows,
                     int cols) {
#pragma omp parallel for
  for (int y = 0; y < rows; ++y) {
    const uint16_t *e = src + (int64_t)y * sstride;
    uint16_t *o = dst + (int64_t)y * dstride;
    uint16_t mmax = e[0];
    for (int x = 1; x < cols; ++x) {
      if (wide(mmax) < wide(e[x])) mmax = e[x];
    }
    uint16_t sum = half_of(0.0f);
    for (int x = 0; x < cols; ++x) {
      o[x] = half_of(expf(wide(half_of(wide(e[x]) - wide(mmax)))));
      sum = half_add(sum, o[x]);
    }
    for (int x = 0; x < cols; ++x) o[x] = half_of(wide(o[x]) / wide(sum));
  }
}

/* SoftmaxGrad on half_t, mshadow/tensor_cpu-inl.h:287-302 */
void orc_softmax_grad_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride,
                          const uint16_t *label, int rows, int cols) {
#pragma omp parallel for
  for (int y = 0; y < rows; ++y) {
    const int k = (int)wide(label[y]);
    const uint16_t *s = src + (int64_t)y * sstride;
    uint16_t *o = dst + (int64_t)y * dstride;
    for (int x = 0; x < cols; ++x) o[x] = (x == k) ? half_of(wide(s[x]) - 1.0f) : s[x];
  }
}

/* SoftmaxGrad with ignore_label, SmoothSoftmaxGrad with and without it,
   mshadow/tensor_cpu-inl.h:304-362. (src - 1.0f) + alpha is evaluated left to right;
   smooth_grad = alpha / (cols - 1) in float. */
static inline void grad_row(float *o, long ostep, const float *s, long sstep, int cols, int k,
                            int flags, int ignored, float alpha, float smooth_grad) {
  for (int x = 0; x < cols; ++x) {
    float v;
    if ((flags & ORC_GRAD_IGNORE) && ignored) {
      v = 0.0f;
    } else if (x == k) {
      v = s[x * sstep] - 1.0f;
      if (flags & ORC_GRAD_SMOOTH) v = v + alpha;
    } else {
      v = s[x * sstep];
      if (flags & ORC_GRAD_SMOOTH) v = v - smooth_grad;
    }
    o[x * ostep] = v;
  }
}

void orc_softmax_grad_ex_f32(float *dst, int dstride, const float *src, int sstride,
                             const float *label, int rows, int cols, int flags,
                             float ignore_label, float alpha) {
  const float smooth_grad = alpha / (float)(cols - 1);
#pragma omp parallel for
  for (int y = 0; y < rows; ++y) {
    const int k = (int)label[y];
    grad_row(dst + (int64_t)y * dstride, 1, src + (int64_t)y * sstride, 1, cols, k, flags,
             (int)ignore_label == k, alpha, smooth_grad);
  }
}

/* Softmax on 3-D tensors, mshadow/tensor_cpu-inl.h:474-495: over the middle dimension,
   max by strict <, exp, sequential sum, true division */
void orc_softmax3d_f32(float *dst, int dstride, const float *src, int sstride, int d0, int d1,
                       int d2) {
#pragma omp parallel for
  for (int y = 0; y < d0; ++y) {
    for (int n = 0; n < d2; ++n) {
      const float *s = src + (int64_t)y * d1 * sstride + n;
      float *o = dst + (int64_t)y * d1 * dstride + n;
      float mmax = s[0];
      for (int x = 1; x < d1; ++x) {
        if (mmax < s[(int64_t)x * sstride]) mmax = s[(int64_t)x * sstride];
      }
      float sum = 0.0f;
      for (int x = 0; x < d1; ++x) {
        o[(int64_t)x * dstride] = expf(s[(int64_t)x * sstride] - mmax);
        sum += o[(int64_t)x * dstride];
      }
      for (int x = 0; x < d1; ++x) o[(int64_t)x * dstride] /= sum;
    }
  }
}

/* the four 3-D gradient functions, mshadow/tensor_cpu-inl.h:364-462 */
void orc_softmax3d_grad_f32(float *dst, int dstride, const float *src, int sstride,
                            const float *label, int lstride, int d0, int d1, int d2, int flags,
                            float ignore_label, float alpha) {
  const float smooth_grad = alpha / (float)(d1 - 1);
#pragma omp parallel for
  for (int n = 0; n < d2; ++n) {
    for (int y = 0; y < d0; ++y) {
      const int k = (int)label[(int64_t)y * lstride + n];
      grad_row(dst + (int64_t)y * d1 * dstride + n, dstride, src + (int64_t)y * d1 * sstride + n,
               sstride, d1, k, flags, k == (int)ignore_label, alpha, smooth_grad);
    }
  }
}

static inline int index_at(const void *index, int is_int, int y) {
  return is_int ? ((const int32_t *)index)[y] : (int)((const float *)index)[y];
}

/* AddTakeGrad, mshadow/tensor_cpu-inl.h:497-508: indices clamped into [0, K), rows added
   one after the other in index order */
void orc_add_take_grad_f32(float *dst, int dstride, int k_rows, const void *index,
                           int index_is_int, int n_index, const float *src, int sstride,
                           int cols) {
  for (int y = 0; y < n_index; ++y) {
    int j = index_at(index, index_is_int, y);
    if (j <= 0) j = 0;
    else if (j >= k_rows) j = k_rows - 1;
    for (int x = 0; x < cols; ++x) dst[(int64_t)j * dstride + x] += src[(int64_t)y * sstride + x];
  }
}

/* AddTakeGradLargeBatch, mshadow/tensor_cpu-inl.h:510-518 */
void orc_add_take_grad_large_batch_f32(float *dst, int dstride, const void *sorted,
                                       const void *index, int index_is_int, int n_index,
                                       const float *src, int sstride, int cols) {
  for (int y = 0; y < n_index; ++y) {
    const int j = index_at(sorted, index_is_int, y);
    const int i = index_at(index, index_is_int, y);
    for (int x = 0; x < cols; ++x) dst[(int64_t)j * dstride + x] += src[(int64_t)i * sstride + x];
  }
}

/* IndexFill, mshadow/tensor_cpu-inl.h:520-528: a later entry of the index overwrites an
   earlier one that names the same row */
void orc_index_fill_f32(float *dst, int dstride, const void *index, int index_is_int,
                        int n_index, const float *src, int sstride, int cols) {
  for (int y = 0; y < n_index; ++y) {
    const int j = index_at(index, index_is_int, y);
    for (int x = 0; x < cols; ++x) dst[(int64_t)j * dstride + x] = src[(int64_t)y * sstride + x];
  }
}

/* ---- the gradient family, the 3-D softmax and the row scatter functions on tensors of another
   element type: type_flag 0 float, 1 double, 2 half_t (mshadow/base.h:305-313 TypeFlag codes).
   The host templates (mshadow/tensor_cpu-inl.h:286-528) are written once for every DType; what
   differs is where a value is rounded. double: `src - 1.0f + alpha` and `src - smooth_grad`
   promote the float operands, smooth_grad itself stays a float quotient. half_t: every operator
   returns a half_t (mshadow/half.h:45-56), so `src - 1.0f` rounds to 16 bits before `+ alpha`
   rounds again; a row addition is one float add rounded to 16 bits. Labels, ignore_label and
   index entries reach `int` through the type's conversion (half_t: through float). */
#define ORC_T_F32 0
#define ORC_T_F64 1
#define ORC_T_F16 2
#define ORC_T_I32 4
#define ORC_T_I64 6

static inline int int_of_entry(const void *v, int type_flag, int64_t i) {
  switch (type_flag) {
    case ORC_T_F32: return (int)((const float *)v)[i];
    case ORC_T_F64: return (int)((const double *)v)[i];
    case ORC_T_F16: return (int)wide(((const uint16_t *)v)[i]);
    case ORC_T_I32: return ((const int32_t *)v)[i];
    default: return (int)((const int64_t *)v)[i];
  }
}

static inline double grad_f64(double p, int at_label, int flags, int ignored, float alpha,
                              float smooth_grad) {
  if ((flags & ORC_GRAD_IGNORE) && ignored) return 0.0;
  if (at_label) {
    double v = p - 1.0f;
    if (flags & ORC_GRAD_SMOOTH) v = v + alpha;
    return v;
  }
  return (flags & ORC_GRAD_SMOOTH) ? p - smooth_grad : p;
}
static inline uint16_t grad_f16(uint16_t p, int at_label, int flags, int ignored, float alpha,
                                float smooth_grad) {
  if ((flags & ORC_GRAD_IGNORE) && ignored) return half_of(0.0f);
  if (at_label) {
    uint16_t v = half_of(wide(p) - 1.0f);
    if (flags & ORC_GRAD_SMOOTH) v = half_of(wide(v) + alpha);
    return v;
  }
  return (flags & ORC_GRAD_SMOOTH) ? half_of(wide(p) - smooth_grad) : p;
}
static inline float grad_f32(float p, int at_label, int flags, int ignored, float alpha,
                             float smooth_grad) {
  if ((flags & ORC_GRAD_IGNORE) && ignored) return 0.0f;
  if (at_label) {
    float v = p - 1.0f;
    if (flags & ORC_GRAD_SMOOTH) v = v + alpha;
    return v;
  }
  return (flags & ORC_GRAD_SMOOTH) ? p - smooth_grad : p;
}

/* d0 == 0: the 2-D functions on rows_or_d1 x cols_or_d2 (label: one per row); otherwise the 3-D
   ones on (d0, d1, d2) with labels (d0, d2) of pitch lstride */
void orc_grad_family_any(int type_flag, void *dst, int dstride, const void *src, int sstride,
                         const void *label, int lstride, int d0, int rows_or_d1, int cols_or_d2,
                         int flags, double ignore_label, float alpha) {
  const int two_d = d0 == 0;
  const int outer = two_d ? rows_or_d1 : d0;
  const int classes = two_d ? cols_or_d2 : rows_or_d1;
  const int inner = two_d ? 1 : cols_or_d2;
  const float smooth_grad = alpha / (float)(unsigned)(classes - 1);
  int ignore_k;
  if (type_flag == ORC_T_F16) ignore_k = (int)wide(half_of((float)ignore_label));
  else if (type_flag == ORC_T_F64) ignore_k = (int)(double)(float)ignore_label;
  else ignore_k = (int)(float)ignore_label;
#pragma omp parallel for
  for (int y = 0; y < outer; ++y) {
    for (int n = 0; n < inner; ++n) {
      const int64_t lab_at = two_d ? y : (int64_t)y * lstride + n;
      const int k = int_of_entry(label, type_flag, lab_at);
      const int ignored = k == ignore_k;
      for (int x = 0; x < classes; ++x) {
        const int64_t so = two_d ? (int64_t)y * sstride + x : ((int64_t)y * classes + x) * sstride + n;
        const int64_t dof = two_d ? (int64_t)y * dstride + x : ((int64_t)y * classes + x) * dstride + n;
        if (type_flag == ORC_T_F16) {
          ((uint16_t *)dst)[dof] = grad_f16(((const uint16_t *)src)[so], x == k, flags, ignored, alpha, smooth_grad);
        } else if (type_flag == ORC_T_F64) {
          ((double *)dst)[dof] = grad_f64(((const double *)src)[so], x == k, flags, ignored, alpha, smooth_grad);
        } else {
          ((float *)dst)[dof] = grad_f32(((const float *)src)[so], x == k, flags, ignored, alpha, smooth_grad);
        }
      }
    }
  }
}

/* Softmax on 3-D tensors of another element type, mshadow/tensor_cpu-inl.h:466-488 */
void orc_softmax3d_any(int type_flag, void *dst, int dstride, const void *src, int sstride, int d0,
                       int d1, int d2) {
  if (type_flag == ORC_T_F32) {
    orc_softmax3d_f32((float *)dst, dstride, (const float *)src, sstride, d0, d1, d2);
    return;
  }
#pragma omp parallel for
  for (int y = 0; y < d0; ++y) {
    for (int n = 0; n < d2; ++n) {
      if (type_flag == ORC_T_F64) {
        const double *s = (const double *)src + (int64_t)y * d1 * sstride + n;
        double *o = (double *)dst + (int64_t)y * d1 * dstride + n;
        double mmax = s[0];
        for (int x = 1; x < d1; ++x) {
          if (mmax < s[(int64_t)x * sstride]) mmax = s[(int64_t)x * sstride];
        }
        double sum = 0.0;
        for (int x = 0; x < d1; ++x) {
          o[(int64_t)x * dstride] = exp(s[(int64_t)x * sstride] - mmax);
          sum += o[(int64_t)x * dstride];
        }
        for (int x = 0; x < d1; ++x) o[(int64_t)x * dstride] /= sum;
      } else {
        const uint16_t *s = (const uint16_t *)src + (int64_t)y * d1 * sstride + n;
        uint16_t *o = (uint16_t *)dst + (int64_t)y * d1 * dstride + n;
        uint16_t mmax = s[0];
        for (int x = 1; x < d1; ++x) {
          if (wide(mmax) < wide(s[(int64_t)x * sstride])) mmax = s[(int64_t)x * sstride];
        }
        uint16_t sum = half_of(0.0f);
        for (int x = 0; x < d1; ++x) {
          const uint16_t t = half_of(expf(wide(half_of(wide(s[(int64_t)x * sstride]) - wide(mmax)))));
          o[(int64_t)x * dstride] = t;
          sum = half_add(sum, t);
        }
        for (int x = 0; x < d1; ++x) {
          o[(int64_t)x * dstride] = half_of(wide(o[(int64_t)x * dstride]) / wide(sum));
        }
      }
    }
  }
}

/* op 0 AddTakeGrad, 1 AddTakeGradLargeBatch, 2 IndexFill (mshadow/tensor_cpu-inl.h:497-528) for
   tables of type_flag elements and index vectors of index_flag entries */
void orc_rows_by_index_any(int op, int type_flag, int index_flag, void *dst, int dstride, int k_rows,
                           const void *sorted, const void *index, int n_index, const void *src,
                           int sstride, int cols) {
  for (int y = 0; y < n_index; ++y) {
    int j, from = y;
    if (op == 0) {
      j = int_of_entry(index, index_flag, y);
      if (j <= 0) j = 0;
      else if (j >= k_rows) j = k_rows - 1;
    } else if (op == 1) {
      j = int_of_entry(sorted, index_flag, y);
      from = int_of_entry(index, index_flag, y);
    } else {
      j = int_of_entry(index, index_flag, y);
    }
    for (int x = 0; x < cols; ++x) {
      const int64_t d = (int64_t)j * dstride + x, s = (int64_t)from * sstride + x;
      if (type_flag == ORC_T_F16) {
        uint16_t *D = (uint16_t *)dst;
        const uint16_t v = ((const uint16_t *)src)[s];
        D[d] = op == 2 ? v : half_of(wide(D[d]) + wide(v));
      } else if (type_flag == ORC_T_F64) {
        double *D = (double *)dst;
        const double v = ((const double *)src)[s];
        D[d] = op == 2 ? v : D[d] + v;
      } else {
        float *D = (float *)dst;
        const float v = ((const float *)src)[s];
        D[d] = op == 2 ? v : D[d] + v;
      }
    }
  }
}

/* SortByKey, mshadow/tensor_cpu-inl.h:531-559: std::stable_sort of the positions under
   keys[a] < keys[b] (ascending) or keys[a] > keys[b] (descending), then keys and values
   permuted alike. Restated as a bottom-up merge sort, which is stable by construction: the
   right run's element is taken only when it is strictly before the left run's. Keys are
   compared in their own type (key_kind 0 float, 1 int32, 2 uint32), so +0.0f and -0.0f are
   equivalent; values are 32-bit words. VectorizedSort (:561-566) is two of these. */
static int key_before(const uint32_t *k, int key_kind, int ascend, int a, int b) {
  if (key_kind == 0) {
    float x, y;
    memcpy(&x, &k[a], 4);
    memcpy(&y, &k[b], 4);
    return ascend ? x < y : x > y;
  }
  if (key_kind == 1) {
    const int32_t x = (int32_t)k[a], y = (int32_t)k[b];
    return ascend ? x < y : x > y;
  }
  return ascend ? k[a] < k[b] : k[a] > k[b];
}
void orc_sort_by_key_32(void *keys, int key_kind, void *values, int n, int is_ascend) {
  if (n <= 0) return;
  uint32_t *k = (uint32_t *)keys, *v = (uint32_t *)values;
  int *ord = (int *)malloc(sizeof(int) * (size_t)n), *tmp = (int *)malloc(sizeof(int) * (size_t)n);
  uint32_t *kc = (uint32_t *)malloc(4 * (size_t)n), *vc = (uint32_t *)malloc(4 * (size_t)n);
  for (int i = 0; i < n; ++i) ord[i] = i;
  for (int64_t width = 1; width < n; width *= 2) {
    for (int64_t lo = 0; lo < n; lo += 2 * width) {
      const int64_t mid = lo + width < n ? lo + width : n, hi = lo + 2 * width < n ? lo + 2 * width : n;
      int64_t i = lo, j = mid, o = lo;
      while (i < mid && j < hi) tmp[o++] = key_before(k, key_kind, is_ascend, ord[j], ord[i]) ? ord[j++] : ord[i++];
      while (i < mid) tmp[o++] = ord[i++];
      while (j < hi) tmp[o++] = ord[j++];
    }
    int *sw = ord; ord = tmp; tmp = sw;
  }
  memcpy(kc, k, 4 * (size_t)n);
  memcpy(vc, v, 4 * (size_t)n);
  for (int i = 0; i < n; ++i) {
    k[i] = kc[ord[i]];
    v[i] = vc[ord[i]];
  }
  free(ord); free(tmp); free(kc); free(vc);
}
void orc_vectorized_sort_32(void *values, int value_kind, void *segments, int n) {
  orc_sort_by_key_32(values, value_kind, segments, n, 1);
  orc_sort_by_key_32(segments, 1, values, n, 1);
}

/* ------------------------------------------------------------------ pool / unpool */

static inline int imin(int a, int b) { return a < b ? a : b; }

/* Plan<PoolingExp>::Eval, mshadow/extension/spatial_pool.h:125-142, driven by the
   MapPlan loop over the flattened output (rows = planes * ph, cols = pw). */
void orc_pool_f32(float *dst, int dstride, const float *src, int sstride, int planes, int h, int w,
                  int ph, int pw, int ky, int kx, int sy, int sx, int reducer) {
  const int out_rows = planes * ph;
#pragma omp parallel for
  for (int i = 0; i < out_rows; ++i) {
    const int py = i % ph;
    const int c = i / ph;
    const int y_start = py * sy;
    const int y_end = imin(y_start + ky, h);
    for (int j = 0; j < pw; ++j) {
      const int x_start = j * sx;
      const int x_end = imin(x_start + kx, w);
      float res = init_f32(reducer);
      for (int y = y_start; y < y_end; ++y) {
        for (int x = x_start; x < x_end; ++x) {
          reduce_f32(&res, src[(int64_t)(c * h + y) * sstride + x], reducer);
        }
      }
      dst[(int64_t)i * dstride + j] = res;
    }
  }
}

/* the same on half_t tensors: red::sum rounds to 16 bits after every add */
void orc_pool_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride, int planes, int h,
                  int w, int ph, int pw, int ky, int kx, int sy, int sx, int reducer) {
  const int out_rows = planes * ph;
#pragma omp parallel for
  for (int i = 0; i < out_rows; ++i) {
    const int py = i % ph;
    const int c = i / ph;
    const int y_start = py * sy;
    const int y_end = imin(y_start + ky, h);
    for (int j = 0; j < pw; ++j) {
      const int x_start = j * sx;
      const int x_end = imin(x_start + kx, w);
      uint16_t res = init_f16(reducer);
      for (int y = y_start; y < y_end; ++y) {
        for (int x = x_start; x < x_end; ++x) {
          reduce_f16(&res, src[(int64_t)(c * h + y) * sstride + x], reducer);
        }
      }
      dst[(int64_t)i * dstride + j] = res;
    }
  }
}

/* Plan<UnPoolingExp>::Eval, mshadow/extension/spatial_unpool.h:102-125: every
   source pixel sums grad over the windows that cover it, weighted by
   PartialGrad(src, pooled) (equality for max / min), py then px ascending. */
void orc_unpool_f32(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                    int pstride, const float *grad, int gstride, int planes, int h, int w, int ph,
                    int pw, int ky, int kx, int sy, int sx, int reducer) {
  const int out_rows = planes * h;
#pragma omp parallel for
  for (int i = 0; i < out_rows; ++i) {
    const int y = i % h;
    const int c = i / h;
    const int py_min = y < ky ? 0 : (y - ky + sy) / sy;
    const int py_max = imin((y + sy) / sy, ph);
    for (int x = 0; x < w; ++x) {
      const float vsrc = src[(int64_t)i * sstride + x];
      const int px_min = x < kx ? 0 : (x - kx + sx) / sx;
      const int px_max = imin((x + sx) / sx, pw);
      float val = 0.0f;
      for (int py = py_min; py < py_max; ++py) {
        for (int px = px_min; px < px_max; ++px) {
          const float p = pooled[(int64_t)(c * ph + py) * pstride + px];
          const float g = grad[(int64_t)(c * ph + py) * gstride + px];
          val += partial_grad_f32(vsrc, p, reducer) * g;
        }
      }
      dst[(int64_t)i * dstride + x] = val;
    }
  }
}

/* ------------------------------------------------------------------ patch2col / col2patch */

/* The index math below is shared by the f16 and f32 entry points through macros so
   that both follow the same lines of the reference.

   Plan<PaddingExp>::Eval, mshadow/extension/pad.h:87-99, over a source with
   (hs, ws) rows / cols per plane: value at padded row i (= plane * (hs + 2 pad_y) + y)
   and column j. */
#define PAD_EVAL(T, ZERO, img, istride, hs, ws, pad_y, pad_x, i, j, out)              \
  do {                                                                                \
    const int new_h_ = (hs) + 2 * (pad_y);                                            \
    const int y_ = (i) % new_h_;                                                      \
    const int c_ = (i) / new_h_;                                                      \
    if (y_ < (pad_y) || (j) < (pad_x)) {                                              \
      (out) = (ZERO);                                                                 \
    } else {                                                                          \
      const int h_ = y_ - (pad_y);                                                    \
      const int w_ = (j) - (pad_x);                                                   \
      if (h_ < (hs) && w_ < (ws)) {                                                   \
        (out) = (img)[(int64_t)(c_ * (hs) + h_) * (istride) + w_];                    \
      } else {                                                                        \
        (out) = (ZERO);                                                               \
      }                                                                               \
    }                                                                                 \
  } while (0)

/* Plan<UnpackPatchToColXExp>::Eval, mshadow/extension/unpack_patch2col.h:126-141,
   with the padded image (pad.h) as its source; output shape per :43-67. */
#define IM2COL_BODY(T, ZERO)                                                          \
  const int hp = h + 2 * pad_y, wp = w + 2 * pad_x;                                   \
  const int o_height = (hp - (dy * (ky - 1) + 1)) / sy + 1;                           \
  const int o_width = (wp - (dx * (kx - 1) + 1)) / sx + 1;                            \
  const int out_rows = ky * kx * c;                                                   \
  const int out_cols = o_height * o_width * n;                                        \
  _Pragma("omp parallel for") for (int i = 0; i < out_rows; ++i) {                    \
    const int x_offset = i % kx * dx;                                                 \
    const int idivp = i / kx;                                                         \
    const int y_offset = idivp % ky * dy;                                             \
    const int ch = idivp / ky;                                                        \
    for (int j = 0; j < out_cols; ++j) {                                              \
      const int x = (j % o_width) * sx + x_offset;                                    \
      const int jdivw = j / o_width;                                                  \
      const int y = (jdivw % o_height) * sy + y_offset;                               \
      const int ni = jdivw / o_height;                                                \
      T v;                                                                            \
      if (x < wp && y < hp) {                                                         \
        PAD_EVAL(T, ZERO, img, istride, h, w, pad_y, pad_x, (ni * c + ch) * hp + y, x, v); \
      } else {                                                                        \
        v = (ZERO);                                                                   \
      }                                                                               \
      col[(int64_t)i * cstride + j] = v;                                              \
    }                                                                                 \
  }

void orc_im2col_f16(uint16_t *col, int cstride, const uint16_t *img, int istride, int n, int c,
                    int h, int w, int ky, int kx, int sy, int sx, int dy, int dx, int pad_y,
                    int pad_x) {
  IM2COL_BODY(uint16_t, (uint16_t)0)
}

void orc_im2col_f32(float *col, int cstride, const float *img, int istride, int n, int c, int h,
                    int w, int ky, int kx, int sy, int sx, int dy, int dx, int pad_y, int pad_x) {
  IM2COL_BODY(float, 0.0f)
}

/* Plan<CroppingExp>::Eval (mshadow/extension/crop.h:103-110, offsets pad_y / pad_x)
   over Plan<PackColToPatchXExp>::Eval (mshadow/extension/pack_col2patch.h:118-144)
   for an image of (n, c, h + 2 pad_y, w + 2 pad_x): patches are visited py then px
   ascending and accumulated in the element type, so half rounds after every add. */
#define COL2IM_BODY(T, ZERO, ADD)                                                     \
  const int hp = h + 2 * pad_y, wp = w + 2 * pad_x;                                   \
  const int o_height = (hp - (dy * (ky - 1) + 1)) / sy + 1;                           \
  const int o_width = (wp - (dx * (kx - 1) + 1)) / sx + 1;                            \
  const int psize_y_dilate = dy * (ky - 1) + 1;                                       \
  const int psize_x_dilate = dx * (kx - 1) + 1;                                       \
  const int out_rows = n * c * h;                                                     \
  _Pragma("omp parallel for") for (int oi = 0; oi < out_rows; ++oi) {                 \
    /* crop: output row oi -> source row of the padded image */                       \
    const int cy = oi % h;                                                            \
    const int cc = oi / h;                                                            \
    const int i = cc * hp + cy + pad_y;                                               \
    const int y = i % hp;                                                             \
    const int idivh = i / hp;                                                         \
    const int ch = idivh % c;                                                         \
    const int ni = idivh / c;                                                         \
    const int py_min = y < psize_y_dilate ? y % dy : (y - psize_y_dilate + sy) / sy;  \
    const int py_max = imin((y + sy) / sy, o_height);                                 \
    for (int oj = 0; oj < w; ++oj) {                                                  \
      const int x = oj + pad_x;                                                       \
      const int px_min = x < psize_x_dilate ? x % dx : (x - psize_x_dilate + sx) / sx; \
      const int px_max = imin((x + sx) / sx, o_width);                                \
      T res = (ZERO);                                                                 \
      for (int py = py_min; py < py_max; py += dy) {                                  \
        for (int px = px_min; px < px_max; px += dx) {                                \
          const int r = (ch * ky + (y - py * sy) / dy) * kx + (x - px * sx) / dx;     \
          const int q = (ni * o_height + py) * o_width + px;                          \
          res = ADD(res, col[(int64_t)r * cstride + q]);                              \
        }                                                                             \
      }                                                                               \
      img[(int64_t)oi * istride + oj] = res;                                          \
    }                                                                                 \
  }

#define ADD_F32(a, b) ((a) + (b))

void orc_col2im_f16(uint16_t *img, int istride, const uint16_t *col, int cstride, int n, int c,
                    int h, int w, int ky, int kx, int sy, int sx, int dy, int dx, int pad_y,
                    int pad_x) {
  COL2IM_BODY(uint16_t, (uint16_t)0, half_add)
}

void orc_col2im_f32(float *img, int istride, const float *col, int cstride, int n, int c, int h,
                    int w, int ky, int kx, int sy, int sx, int dy, int dx, int pad_y, int pad_x) {
  COL2IM_BODY(float, 0.0f, ADD_F32)
}
