/*
 * Which terms of a left-to-right binary16 sum of non-negative terms can be left out.
 *
 * In `sum += t` on half_t (mshadow/half.h:58-62: widen, add, round back) a term below half an
 * ulp of the sum changes nothing: S + t lies strictly between S and the midpoint to the next
 * binary16 number and rounds back to S. The sum of non-negative terms never decreases, so a
 * lower bound `low` of the sum in front of a term - the largest term already added is one -
 * gives a bound for the whole rest of the row: every term below half an ulp of `low` is a
 * no-op wherever it stands behind that point. A softmax row of 32000 terms keeps a few
 * thousand; the others need not enter the chain of dependent adds at all. Ties (a term of
 * exactly half an ulp) and everything larger stay in; so do NaN terms.
 *
 * Plain integer arithmetic on bit patterns, usable on the host and on the device.
 */
#ifndef MSHADOW_HIP_KERNELS_HALF_PRUNE_H_
#define MSHADOW_HIP_KERNELS_HALF_PRUNE_H_

#include <stdint.h>

#include "../../base.h"

namespace mshadow {
namespace hip {

/*! \brief smallest bit pattern of a non-negative binary16 term that may still change a sum
 *  that is at least `low_bits` (a non-negative binary16 bit pattern): half an ulp of `low`,
 *  i.e. 2^(e - 26) for a normal `low` with biased exponent e, and the smallest subnormal for a
 *  subnormal or zero `low` (only a zero term is certain to change nothing there). A term whose
 *  pattern compares below the result, as an unsigned integer, is a no-op. */
MSHADOW_XINLINE uint32_t HalfSignificantFrom(uint32_t low_bits) {
  const uint32_t e = (low_bits >> 10) & 0x1fu;
  if (e < 2u) return 1u;                       // half an ulp is below the smallest subnormal
  if (e >= 12u) return (e - 11u) << 10;        // 2^(e - 26) is a normal number
  return 1u << (e - 2u);                       // 2^(e - 26) = 2^-24 * 2^(e - 2), subnormal
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_HALF_PRUNE_H_
