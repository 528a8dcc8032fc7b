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
 * associative: lanes quantise their terms, a wave/block sums the integers (held in
 * floats, exact below 2^24), and the chunk is accepted if m + sum(q) stays below 2^24
 * and no term was a tie. Otherwise
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

/*! \brief quantised contributions are carried as floats holding integers: sums below
 *  2^24 are exact, and a sum that reaches 2^24 in exact arithmetic can never round to
 *  less, so "not below kLimit" is a faithful overflow test. A lane that must not be
 *  accepted as integers (tie, inf, NaN, unusable binade) contributes kReject. */
const float kLimit = 16777216.0f;  // 2^24
const float kReject = 33554432.0f;  // 2^25

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
  float m;        //!< S / u, an integer in [2^23, 2^24), as a float
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
  r.m = r.usable ? s * r.inv_u : 0.0f;  /* exact: scaling by a power of two */
  return r;
}

/*! \brief contribution of one lane's N consecutive terms: sum of rne(t / u), or kReject
 *  if any term is a tie (or NaN). Terms too large for the binade simply make the sum
 *  reach kLimit. When the binade is not usable (S is 0, subnormal-small, inf or NaN)
 *  only all-zero lanes can be accepted: adding +0 never changes S. */
template <int N>
OSUM_HD float LaneQuant(const float (&t)[N], const Binade &b) {
  if (!b.usable) {
    bool any = false;
    for (int i = 0; i < N; ++i) any = any || !(t[i] == 0.0f);
    return any ? kReject : 0.0f;
  }
  float sum = 0.0f;
  float worst = 0.0f;    /* largest distance of a scaled term from its rounded value */
  float least = 0.0f;    /* most negative scaled term */
  for (int i = 0; i < N; ++i) {
    const float scaled = t[i] * b.inv_u;  /* exact: inv_u is a power of two */
    const float q = rintf(scaled);        /* round to nearest even */
    worst = fmaxf(worst, fabsf(scaled - q));
    least = fminf(least, scaled);
    sum += q;
  }
  /* worst == 0.5 exactly when some term sits half way between two integers. A negative
     term would move the sum down, which the one-sided Fits() does not watch. NaN and
     infinite terms slip through the max / min but leave `sum` NaN or infinite, which
     no caller accepts (every acceptance is a `< kLimit` comparison). */
  const bool bad = !(worst < 0.5f) || least < 0.0f;
  return bad ? kReject : sum;
}

/*! \brief true if integer contributions totalling q can be added without leaving the
 *  binade (written so that NaN fails) */
OSUM_HD bool Fits(const Binade &b, float q) { return b.m + q < kLimit; }

/*! \brief S after accepting integer contributions summing to q (Fits(b, q) holds) */
OSUM_HD float Accept(float s, const Binade &b, float q) {
  return b.usable ? (b.m + q) * b.u : s;
}

/* ---- whole-row planning -------------------------------------------------------------
 * A row is cut into chunks (the terms one wave holds in one register slab). Cheap
 * approximate prefix sums say, before any exact work, which chunks the running sum
 * traverses without leaving a binade ("clean"): those are quantised against that binade
 * by all waves at once and enter the sum as one exact integer each. Only the chunks in
 * which a power of two is crossed ("dirty", about one per binade of the final sum) are
 * walked in order, and inside such a chunk the same plan is made per lane: lanes that
 * stay in one binade enter as integers, the few next to the crossing (and lanes holding
 * a tie) are added term by term. The plan is only a plan: every clean run is verified
 * when it is applied (FlushRun), so a wrong guess costs time, never a bit. */

/*! \brief plan codes: a biased exponent e (27 <= e < 255) means clean in that binade;
 *  kPlanTwoBinades + e: the sum starts in binade e and may cross into e + 1 (or holds a
 *  tie): walked with both quantisations prepared; kPlanWalk: anything else */
const int kPlanWalk = -1;
const int kPlanTwoBinades = 256;

OSUM_HD uint32_t ExponentOf(float f) { return (BitsOf(f) >> 23) & 0xffu; }

/*! \brief how far the sequential sum of n non-negative terms can sit from an accurate
 *  sum of the same terms, relative to it: every addition rounds by at most half an ulp
 *  of the running sum (n * 2^-25 in all, and rows with many terms below half an ulp come
 *  close to it); doubled for the approximate sums themselves */
OSUM_HD float PlanMargin(int n) {
  const float m = static_cast<float>(n) * 5.9604644775390625e-08f;  // n * 2^-24
  return m < 1.52587890625e-05f ? 1.52587890625e-05f : (m > 0.25f ? 0.25f : m);
}

/*! \brief binade with biased exponent e (27 <= e < 255); m is not set */
OSUM_HD Binade BinadeOfExponent(uint32_t e) {
  Binade r;
  r.usable = true;
  r.u = FloatOf((e - 23u) << 23);
  r.inv_u = FloatOf((277u - e) << 23);
  r.m = 0.0f;
  return r;
}

/*! \brief plan for a piece (a chunk, or one lane's terms) whose approximate prefix sums
 *  before / after are st <= en: the binade it stays in, or kPlanWalk */
OSUM_HD int PlanPiece(float st, float en, float margin) {
  const float lo = st * (1.0f - margin);
  const float hi = en * (1.0f + margin);
  /* 2^-98: keeps the exponent of lo at 28 or more; comparisons are false for NaN */
  const bool usable = lo >= 3.1554436e-30f && hi < 1.0e38f;
  const int elo = static_cast<int>(ExponentOf(lo));
  const int ehi = static_cast<int>(ExponentOf(hi));
  if (!usable) return kPlanWalk;
  if (elo == ehi) return elo;
  return (ehi == elo + 1) ? kPlanTwoBinades + elo : kPlanWalk;
}
/*! \brief the same for one lane's few terms, where only "stays in a binade" is of use */
OSUM_HD int PlanLane(float st, float en, float margin) {
  const int c = PlanPiece(st, en, margin);
  return c < kPlanTwoBinades ? c : kPlanWalk;
}

/*! \brief apply a run of clean pieces - integer contributions totalling `run`, quantised
 *  against the binade with biased exponent e_run - to s. Sets *fail (and returns s
 *  unchanged) unless s really is in that binade and stays in it. */
OSUM_HD float FlushRun(float s, int e_run, uint32_t run, bool *fail) {
  const Binade b = BinadeOfExponent(static_cast<uint32_t>(e_run));
  const float m = s * b.inv_u;  /* s in the binade <=> 2^23 <= m < 2^24, and m is an integer */
  const float r = m + static_cast<float>(run);
  const bool ok = m >= 8388608.0f && r < kLimit && run < 16777216u;
  if (!ok) *fail = true;
  return ok ? r * b.u : s;
}

/*! \brief the real thing: N float additions in order */
template <int N>
OSUM_HD float TrueAdd(float s, const float (&t)[N]) {
  for (int i = 0; i < N; ++i) s = s + t[i];
  return s;
}

/* ---- the row as a list of addends -------------------------------------------------------
 * The planned row sum of softmax_kernels.h turns a row into a short ordered list of float
 * addends whose plain serial sum IS the left-to-right sum of all terms: a lane (N consecutive
 * terms) whose running sum provably stays in one binade joins a run of such lanes, and the
 * run enters the list as ONE addend, its integer total times the binade's ulp; any other lane
 * (next to a power of two, or holding a tie) enters with its N terms themselves. Adding a
 * run's addend is exact when the sum is in the run's binade before and after it, which is
 * checked on the sums actually obtained (RunHolds): a wrong plan is noticed, never used. */

/*! \brief quantisation of one lane's N non-negative terms against the binade with biased
 *  exponent e (0 = the subnormal range, where sums are exact): two accumulators start at
 *  the bottom of the binade, one ulp apart, and take the terms by ordinary float additions.
 *  While both stay in the binade each addition moves them by rne(t / ulp) ulps; a term that
 *  lies half way between two multiples of the ulp moves the even one down and the odd one
 *  up, so the accumulators end one ulp apart exactly when no term was a tie. */
struct LaneQuantum {
  uint32_t q;  //!< sum of rne(t / ulp) over the lane's terms
  bool ok;     //!< no tie, no NaN, and the lane alone does not leave the binade
};
template <int N>
OSUM_HD LaneQuantum LaneDualQuant(const float (&t)[N], uint32_t e) {
  const uint32_t base = e << 23;
  float lo = FloatOf(base), hi = FloatOf(base + 1u);
  for (int i = 0; i < N; ++i) {
    lo = lo + t[i];
    hi = hi + t[i];
  }
  const uint32_t blo = BitsOf(lo), bhi = BitsOf(hi);
  LaneQuantum r;
  r.ok = (bhi - blo == 1u) && blo >= base && bhi < base + (1u << 23);
  r.q = blo - base;
  return r;
}

/*! \brief bounds on the sequential sum from an accurate sum `approx` of the same terms:
 *  every addition rounds by at most half an ulp, so after n terms the sequential sum sits
 *  within n * 2^-24 of it (relative); sums of softmax terms stay well inside a quarter of
 *  that below and almost nothing above. The bounds only steer the plan. */
OSUM_HD float PlanLowBound(float approx, float terms_in_front) {
  return approx * (1.0f - (terms_in_front * 1.4901161193847656e-08f + 8.0e-6f));  // n * 2^-26
}
OSUM_HD float PlanHighBound(float approx) { return approx * (1.0f + 8.0e-6f); }

/*! \brief the binade a piece stays in if the sum is at least `low` in front of it and at
 *  most `high` behind it; -1 if those lie in different binades (or are not finite) */
OSUM_HD int PlanBinade(float low, float high) {
  const uint32_t blo = BitsOf(low), bhi = BitsOf(high);
  const uint32_t elo = (blo >> 23) & 0xffu, ehi = (bhi >> 23) & 0xffu;
  const bool ok = elo == ehi && ehi < 255u && ((blo | bhi) >> 31) == 0u;
  return ok ? static_cast<int>(elo) : -1;
}

/*! \brief the addend of a run with integer total r in binade e. A total that cannot fit
 *  (the sum itself takes at least 2^23 ulps) becomes an addend that carries any sum out
 *  of the binade, so that RunHolds fails. */
OSUM_HD float RunAddend(uint32_t e, uint32_t r) {
  const uint32_t base = e << 23;
  return r < (1u << 23) ? FloatOf(base + r) - FloatOf(base) : FloatOf(base + (1u << 23));
}

/*! \brief was adding a run of binade e exact? (the sum before and after lies in it) */
OSUM_HD bool RunHolds(float before, float after, uint32_t e) {
  const uint32_t bb = BitsOf(before), ba = BitsOf(after);
  return (bb >> 23) == e && (ba >> 23) == e;  // sign bits are part of the comparison
}

}  // namespace ordered_sum
#endif  // MSHADOW_AMD_CSRC_ORDERED_SUM_H_
