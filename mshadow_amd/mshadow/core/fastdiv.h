/*
 * Division of a 31-bit index by a divisor known only at launch time, as one multiply-high
 * and one shift. A hardware integer division costs the GPU some forty instructions; index
 * math that splits a flat offset into (row, column) pays it per element otherwise.
 */
#ifndef MSHADOW_CORE_FASTDIV_H_
#define MSHADOW_CORE_FASTDIV_H_

#include <stdint.h>

#include "./config.h"

namespace mshadow {

/*! \brief floor(e / d) for 0 <= e < 2^31 and d >= 1.
 *  With p = 31 + ceil(log2 d) and mul = ceil(2^p / d) (which fits 32 bits for d > 1),
 *  floor(e * mul / 2^p) equals floor(e / d) over that range: the excess of mul over
 *  2^p / d is below 1 / d of a unit per 2^31 of e. */
struct FastDivU32 {
  uint32_t mul;
  uint32_t shift;
  uint32_t div;
  FastDivU32() : mul(0), shift(0), div(1) {}
  explicit FastDivU32(uint32_t d) : mul(0), shift(0), div(d) {
    if (d > 1) {
      uint32_t lg = 0;
      while ((1ull << lg) < d) ++lg;
      const uint32_t p = 31 + lg;
      mul = static_cast<uint32_t>(((1ull << p) + d - 1) / d);
      shift = p - 32;
    }
  }
  /*! \brief e % d */
  MSHADOW_XINLINE uint32_t Mod(uint32_t e) const { return e - Div(e) * div; }
  MSHADOW_XINLINE uint32_t Div(uint32_t e) const {
    if (div == 1) return e;
#if defined(__HIP_DEVICE_COMPILE__)
    return __umulhi(e, mul) >> shift;
#else
    return static_cast<uint32_t>((static_cast<uint64_t>(e) * mul) >> 32) >> shift;
#endif
  }
};

}  // namespace mshadow
#endif  // MSHADOW_CORE_FASTDIV_H_
