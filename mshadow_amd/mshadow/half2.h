/*
 * half2_t: two binary16 values that move and compute together.
 *
 * Contract: mshadow/half2.h:22-143 of the reference, where the type wraps CUDA's half2 in
 * device code of sm_53 and later and is a pair of half_t everywhere else. Here it is the pair
 * of half_t on both sides of the compilation: every operator is half_t's, lane by lane (each
 * result rounded to binary16 once), which is also what the reference's device form computes
 * (it widens both lanes to float, operates and rounds back). 4 bytes, 4-byte aligned, so a
 * tensor of half2_t is a tensor of half_t with half as many columns.
 */
#ifndef MSHADOW_HALF2_H_
#define MSHADOW_HALF2_H_

#include <math.h>

#include "./half.h"

namespace mshadow {
namespace half {

class MSHADOW_ALIGNED(4) half2_t {
 public:
  /*! \brief the lanes; the member keeps the name callers of the reference use */
  half_t half_t2[2];

  MSHADOW_XINLINE half2_t() {}
  MSHADOW_XINLINE half2_t(const half2_t &o) { Set(o.half_t2[0], o.half_t2[1]); }
  MSHADOW_XINLINE explicit half2_t(half_t lo, half_t hi) { Set(lo, hi); }
  /*! \brief the same integer in both lanes */
  MSHADOW_XINLINE explicit half2_t(int both) { Set(static_cast<half_t>(both), static_cast<half_t>(both)); }

  MSHADOW_XINLINE half2_t operator=(const half2_t &o) {
    Set(o.half_t2[0], o.half_t2[1]);
    return o;
  }
  MSHADOW_XINLINE half2_t operator+() { return *this; }
  MSHADOW_XINLINE half2_t operator-() { return half2_t(-half_t2[0], -half_t2[1]); }
  /* a op= b for anything `half2_t op b` is defined for */
  template <typename T>
  MSHADOW_XINLINE half2_t operator+=(const T &b) { return *this = half2_t(*this + b); }
  template <typename T>
  MSHADOW_XINLINE half2_t operator-=(const T &b) { return *this = half2_t(*this - b); }
  template <typename T>
  MSHADOW_XINLINE half2_t operator*=(const T &b) { return *this = half2_t(*this * b); }
  template <typename T>
  MSHADOW_XINLINE half2_t operator/=(const T &b) { return *this = half2_t(*this / b); }

 private:
  MSHADOW_XINLINE void Set(half_t lo, half_t hi) {
    half_t2[0] = lo;
    half_t2[1] = hi;
  }
};

/* the four arithmetic operators, lane by lane in half_t */
#define MSHADOW_HALF2_LANEWISE(OP)                                                    \
  MSHADOW_XINLINE half2_t operator OP(half2_t a, half2_t b) {                         \
    return half2_t(a.half_t2[0] OP b.half_t2[0], a.half_t2[1] OP b.half_t2[1]);      \
  }
MSHADOW_HALF2_LANEWISE(+)
MSHADOW_HALF2_LANEWISE(-)
MSHADOW_HALF2_LANEWISE(*)
MSHADOW_HALF2_LANEWISE(/)
#undef MSHADOW_HALF2_LANEWISE

/*! \brief floating-point remainder of each lane, computed in float */
MSHADOW_XINLINE half2_t operator%(half2_t a, half2_t b) {
  const float lo = ::fmodf(static_cast<float>(a.half_t2[0]), static_cast<float>(b.half_t2[0]));
  const float hi = ::fmodf(static_cast<float>(a.half_t2[1]), static_cast<float>(b.half_t2[1]));
  return half2_t(half_t(lo), half_t(hi));
}
/*! \brief true when both lanes compare equal */
MSHADOW_XINLINE bool operator==(half2_t a, half2_t b) {
  return a.half_t2[0] == b.half_t2[0] && a.half_t2[1] == b.half_t2[1];
}

}  // namespace half
}  // namespace mshadow
#endif  // MSHADOW_HALF2_H_
