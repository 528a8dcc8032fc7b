/*
 * Parallel evaluation of a strictly left-to-right float32 sum of non-negative terms.
 *
 * The CPU softmax of the reference adds exp(x - max) into one float accumulator in
 * column order (mshadow/tensor_cpu-inl.h:277-281). With 32000 terms that running sum
 * sits 2.6e-5 (relative) below the exact sum, more than the 1e-5 the results must
 * agree to, so an accurate tree sum does not reproduce it. This file reproduces it
 * bit for bit, in parallel, from one observation:
 *
 *   while the accumulator S stays inside one binade [2^k, 2^(k+1)), its ulp
 *   u = 2^(k-23) is constant and S = m*u with integer m. For a term t >= 0 with
 *   S + t < 2^(k+1),   fl(S + t) = u * (m + rne(t / u))   unless t/u lies exactly
 *   half way between two integers (then the tie-break depends on the parity of m).
 *
 * So inside a binade the float adds are exact INTEGER adds of q = rne(t/u), which are
 * associative: lanes quantise their terms, a wave/block sums the integers, and the
 * chunk is accepted if m + sum(q) stays below 2^24 and no term was a tie. Otherwise
 * the first offending position is located by prefix sums; everything before it is
 * accepted, the offending lane performs its (at most 4) additions as real float adds,
 * and the remainder is re-quantised against the new binade. A row of N(0,3) logits
 * crosses about twenty binades, nearly all of them within its first few hundred terms.
 *
 * The per-lane arithmetic below is plain C++ (no intrinsics besides rintf) so that a
 * host program can exercise it lane by lane; the wave / block collectives live in
 * softmax_kernels.h.
 */
#ifndef MSHADOW_AMD_CSRC_ORDERED_SUM_H_
#define MSHADOW_AMD_CSRC_ORDERED_SUM_H_

#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define OSUM_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define OSUM_HD inline __attribute__((always_inline))
#endif

namespace ordered_sum {

/*! \brief a quantised contribution this large means "do not accept me as an integer" */
const uint32_t kBig = 1u << 24;

OSUM_HD uint32_t BitsOf(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof(u));
  return u;
}
OSUM_HD float FloatOf(uint32_t u) {
  float f;
  memcpy(&f, &u, sizeof(f));
  return f;
}

/*! \brief the binade of the running sum S >= 0 */
struct Binade {
  float u;        //!< ulp of S: 2^(k-23)
  float inv_u;    //!< 2^(23-k)
  uint32_t m;     //!< S / u, an integer in [2^23, 2^24)
  bool usable;    //!< S is a positive normal number large enough for u and inv_u to be normal
};

OSUM_HD Binade BinadeOf(float s) {
  const uint32_t b = BitsOf(s);
  const uint32_t e = (b >> 23) & 0xffu;
  Binade r;
  /* e >= 27 keeps u = 2^(e-150) normal; e < 255 excludes inf / NaN; sign bit must be 0 */
  r.usable = (b >> 31) == 0 && e >= 27u && e < 255u;
  r.u = r.usable ? FloatOf((e - 23u) << 23) : 0.0f;
  r.inv_u = r.usable ? FloatOf((277u - e) << 23) : 0.0f;
  r.m = r.usable ? ((b & 0x7fffffu) | 0x800000u) : 0u;
  return r;
}

/*! \brief rne(t / u) of one term, or kBig if the term is a tie, too large, inf or NaN */
OSUM_HD uint32_t QuantOne(float t, float inv_u) {
  const float scaled = t * inv_u;  /* exact: inv_u is a power of two */
  if (!(scaled < 16777216.0f)) return kBig;
  const float q = rintf(scaled);   /* round to nearest even */
  if (fabsf(scaled - q) == 0.5f) return kBig;
  return static_cast<uint32_t>(q);
}

/*! \brief contribution of one lane's N consecutive terms, saturated at kBig.
 *  When the binade is not usable (S is 0, subnormal-small, inf or NaN) only all-zero
 *  lanes can be accepted: adding +0 never changes S. */
template <int N>
OSUM_HD uint32_t LaneQuant(const float (&t)[N], const Binade &b) {
  if (!b.usable) {
    bool any = false;
    for (int i = 0; i < N; ++i) any = any || !(t[i] == 0.0f);
    return any ? kBig : 0u;
  }
  uint32_t s = 0;
  for (int i = 0; i < N; ++i) s += QuantOne(t[i], b.inv_u);
  return s < kBig ? s : kBig;
}

/*! \brief S after accepting integer contributions summing to q (m + q < 2^24) */
OSUM_HD float Accept(float s, const Binade &b, uint32_t q) {
  return b.usable ? static_cast<float>(b.m + q) * b.u : s;
}

/*! \brief the real thing: N float additions in order */
template <int N>
OSUM_HD float TrueAdd(float s, const float (&t)[N]) {
  for (int i = 0; i < N; ++i) s = s + t[i];
  return s;
}

}  // namespace ordered_sum
#endif  // MSHADOW_AMD_CSRC_ORDERED_SUM_H_
