/*
 * half::half_t - IEEE binary16 storage type of the mshadow API.
 *
 * Semantics follow mshadow/half.h:45-66 and :94-351 of the reference: the value is
 * held as 16 raw bits; every arithmetic or comparison operator widens both operands
 * to float, computes in float and (for arithmetic) rounds the result back to half
 * with round-to-nearest-even, so `a += b` rounds after each step. On gfx950 the two
 * conversions are the hardware v_cvt instructions reached through _Float16; on the
 * host they are F16C where the compiler enables it and integer code otherwise. All
 * three agree bit for bit on non-NaN inputs.
 */
#ifndef MSHADOW_HALF_H_
#define MSHADOW_HALF_H_

#include <stdint.h>
#include <string.h>

#include "./core/config.h"

#if !defined(__HIP_DEVICE_COMPILE__) && defined(__F16C__)
#include <immintrin.h>
#define MSHADOW_HALF_HOST_F16C 1
#else
#define MSHADOW_HALF_HOST_F16C 0
#endif

namespace mshadow {
namespace half {

namespace detail {
/*! \brief float -> half bits, round to nearest even, integer-only host fallback */
MSHADOW_XINLINE uint16_t EncodeSoft(float value) {
  uint32_t x;
  memcpy(&x, &value, sizeof(x));
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t mag = x & 0x7fffffffu;
  if (mag > 0x7f800000u) return static_cast<uint16_t>(sign | 0x7e00u | ((mag >> 13) & 0x1ffu));
  if (mag >= 0x38800000u) {  // at least the smallest normal half
    const uint32_t rounded = mag + 0xfffu + ((mag >> 13) & 1u);
    uint32_t h = (rounded - 0x38000000u) >> 13;
    if (h > 0x7c00u) h = 0x7c00u;
    return static_cast<uint16_t>(sign | h);
  }
  const uint32_t e = mag >> 23;
  if (e < 102u) return static_cast<uint16_t>(sign);  // below half of the smallest subnormal
  const uint32_t m = (mag & 0x7fffffu) | 0x800000u;
  const uint32_t sh = 126u - e;
  uint32_t q = m >> sh;
  const uint32_t rem = m & ((1u << sh) - 1u);
  const uint32_t mid = 1u << (sh - 1u);
  if (rem > mid || (rem == mid && (q & 1u))) ++q;
  return static_cast<uint16_t>(sign | q);
}
/*! \brief half bits -> float, exact */
MSHADOW_XINLINE float DecodeSoft(uint16_t h) {
  const uint32_t sign = (static_cast<uint32_t>(h) & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 0x1fu;
  const uint32_t m = h & 0x3ffu;
  uint32_t x;
  if (e == 0) {
    float f = static_cast<float>(m) * 5.9604644775390625e-08f;  // m * 2^-24
    memcpy(&x, &f, sizeof(x));
    x |= sign;
  } else if (e == 31) {
    x = sign | 0x7f800000u | (m << 13);
  } else {
    x = sign | ((e + 112u) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &x, sizeof(f));
  return f;
}
MSHADOW_XINLINE uint16_t Encode(float value) {
#if defined(__HIP_DEVICE_COMPILE__)
  _Float16 h = static_cast<_Float16>(value);  // v_cvt_f16_f32, round to nearest even
  uint16_t bits;
  __builtin_memcpy(&bits, &h, sizeof(bits));
  return bits;
#elif MSHADOW_HALF_HOST_F16C
  return static_cast<uint16_t>(_cvtss_sh(value, 0));
#else
  return EncodeSoft(value);
#endif
}
MSHADOW_XINLINE float Decode(uint16_t bits) {
#if defined(__HIP_DEVICE_COMPILE__)
  _Float16 h;
  __builtin_memcpy(&h, &bits, sizeof(bits));
  return static_cast<float>(h);
#elif MSHADOW_HALF_HOST_F16C
  return _cvtsh_ss(bits);
#else
  return DecodeSoft(bits);
#endif
}
}  // namespace detail

class MSHADOW_ALIGNED(2) half_t {
 public:
  /*! \brief raw IEEE binary16 bits */
  uint16_t half_;

  /*! \brief build from a bit pattern */
  static MSHADOW_XINLINE half_t Binary(uint16_t value) {
    half_t r;
    r.half_ = value;
    return r;
  }
  MSHADOW_XINLINE half_t() {}
  MSHADOW_XINLINE half_t(const float &v) : half_(detail::Encode(v)) {}  // NOLINT(*)
  MSHADOW_XINLINE explicit half_t(const double &v) : half_(detail::Encode(static_cast<float>(v))) {}
  MSHADOW_XINLINE explicit half_t(const int8_t &v) : half_(detail::Encode(static_cast<float>(v))) {}
  MSHADOW_XINLINE explicit half_t(const uint8_t &v) : half_(detail::Encode(static_cast<float>(v))) {}
  MSHADOW_XINLINE explicit half_t(const int32_t &v) : half_(detail::Encode(static_cast<float>(v))) {}
  MSHADOW_XINLINE explicit half_t(const uint32_t &v) : half_(detail::Encode(static_cast<float>(v))) {}
  MSHADOW_XINLINE explicit half_t(const int64_t &v) : half_(detail::Encode(static_cast<float>(v))) {}
  MSHADOW_XINLINE explicit half_t(const uint64_t &v) : half_(detail::Encode(static_cast<float>(v))) {}

  MSHADOW_XINLINE operator float() const { return detail::Decode(half_); }  // NOLINT(*)
  MSHADOW_XINLINE operator float() const volatile { return detail::Decode(half_); }  // NOLINT(*)

#define MSHADOW_HALF_COMPOUND(AOP, OP)                                        \
  template <typename T>                                                       \
  MSHADOW_XINLINE half_t operator AOP(const T &a) {                           \
    return *this = half_t(static_cast<float>(*this) OP static_cast<float>(a)); \
  }                                                                           \
  template <typename T>                                                       \
  MSHADOW_XINLINE half_t operator AOP(const volatile T &a) volatile {         \
    return *this = half_t(static_cast<float>(*this) OP static_cast<float>(a)); \
  }
  MSHADOW_HALF_COMPOUND(+=, +)
  MSHADOW_HALF_COMPOUND(-=, -)
  MSHADOW_HALF_COMPOUND(*=, *)
  MSHADOW_HALF_COMPOUND(/=, /)
#undef MSHADOW_HALF_COMPOUND

  MSHADOW_XINLINE half_t operator+() { return *this; }
  MSHADOW_XINLINE half_t operator-() { return half_t(-static_cast<float>(*this)); }

  MSHADOW_XINLINE half_t operator=(const half_t &a) {
    half_ = a.half_;
    return a;
  }
  template <typename T>
  MSHADOW_XINLINE half_t operator=(const T &a) {
    return *this = half_t(a);
  }
  MSHADOW_XINLINE half_t operator=(const half_t &a) volatile {
    half_ = a.half_;
    return a;
  }
  template <typename T>
  MSHADOW_XINLINE half_t operator=(const T &a) volatile {
    return *this = half_t(a);
  }
};

#define MSHADOW_HALF_BINARY(RTYPE, OP)                                \
  MSHADOW_XINLINE RTYPE operator OP(half_t a, half_t b) {             \
    return RTYPE(static_cast<float>(a) OP static_cast<float>(b));     \
  }                                                                   \
  template <typename T>                                               \
  MSHADOW_XINLINE RTYPE operator OP(half_t a, T b) {                  \
    return RTYPE(static_cast<float>(a) OP static_cast<float>(b));     \
  }                                                                   \
  template <typename T>                                               \
  MSHADOW_XINLINE RTYPE operator OP(T a, half_t b) {                  \
    return RTYPE(static_cast<float>(a) OP static_cast<float>(b));     \
  }
MSHADOW_HALF_BINARY(half_t, +)
MSHADOW_HALF_BINARY(half_t, -)
MSHADOW_HALF_BINARY(half_t, *)
MSHADOW_HALF_BINARY(half_t, /)
MSHADOW_HALF_BINARY(bool, >)
MSHADOW_HALF_BINARY(bool, <)
MSHADOW_HALF_BINARY(bool, >=)
MSHADOW_HALF_BINARY(bool, <=)
MSHADOW_HALF_BINARY(bool, ==)
MSHADOW_HALF_BINARY(bool, !=)
#undef MSHADOW_HALF_BINARY

/*! \brief most negative / most positive finite half (mshadow/half.h:350-351) */
#define MSHADOW_HALF_MIN mshadow::half::half_t::Binary(0xFBFF);
#define MSHADOW_HALF_MAX mshadow::half::half_t::Binary(0x7BFF);

}  // namespace half
}  // namespace mshadow
#endif  // MSHADOW_HALF_H_
