// The pruning rule of the binary16 softmax row sum (mshadow/hip/kernels/half_prune.h), checked
// exhaustively: for EVERY pair of a finite non-negative binary16 sum S and a finite non-negative
// binary16 term t, if the rule calls t a no-op against a lower bound low <= S, then half_t's
// `S += t` (widen to float, add, round to nearest even back to binary16) must return S. The
// bound is monotone in `low`, so it is enough to check low == S and that monotony.
// Prints "OK <pairs the rule drops> <no-op pairs it keeps>" and exits 0.
#include <immintrin.h>

#include <cstdint>
#include <cstdio>

#include <mshadow/hip/kernels/half_prune.h>

static inline float Widen(uint16_t h) { return _cvtsh_ss(h); }
static inline uint16_t Narrow(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT); }

int main() {
  using mshadow::hip::HalfSignificantFrom;
  uint32_t prev = 0;
  for (uint32_t s = 0; s <= 0x7c00u; ++s) {  // monotone, +inf included
    const uint32_t from = HalfSignificantFrom(s);
    if (from < prev || from == 0u) {
      std::printf("FAIL not monotone at %04x\n", s);
      return 1;
    }
    prev = from;
  }
  unsigned long long dropped = 0, kept_noops = 0;
  for (uint32_t s = 0; s <= 0x7bffu; ++s) {
    const uint32_t from = HalfSignificantFrom(s);
    const float wide = Widen(static_cast<uint16_t>(s));
    for (uint32_t t = 0; t <= 0x7bffu; ++t) {
      const uint16_t r = Narrow(wide + Widen(static_cast<uint16_t>(t)));
      if (t < from) {
        ++dropped;
        if (r != s) {
          std::printf("FAIL S=%04x t=%04x: dropped, but S + t = %04x\n", s, t, r);
          return 1;
        }
      } else if (r == s) {
        ++kept_noops;
      }
    }
  }
  std::printf("OK %llu %llu\n", dropped, kept_noops);
  return 0;
}
