/*
 * Random numbers on the device: Philox-4x32-10, a counter-based generator (Salmon, Moraes,
 * Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11). Element e of a call
 * is a pure function of (seed, subsequence, counter + e / 4, e % 4), so a launch needs no
 * generator state in memory and any launch shape gives the same values; the caller (the
 * Random<gpu> object) advances `counter` by the blocks a call consumed.
 *
 * This is the role cuRAND's default generator plays for Random<gpu> in the reference
 * (mshadow/random.h:372-568: curandGenerate / curandGenerateUniform /
 * curandGenerateNormal). The values are those of Philox, not of cuRAND's XORWOW: no two
 * generator families agree, and the reference's CPU path (std::mt19937) does not agree
 * with its own GPU path either.
 *   uniform  u = ((x >> 9) + 0.5) * 2^-23, strictly inside (0, 1), then u * (b - a) + a
 *   normal   Box-Muller on two uniforms: sqrt(-2 ln u1) * (cos, sin)(2 pi u2), then
 *            mu + z * sigma
 * Double tensors (Random<gpu, double>, mshadow/random.h:486-514 of the reference:
 * curandGenerateUniformDouble / curandGenerateNormalDouble) take two words per value:
 *   uniform  n = word0 * 2^20 + (word1 >> 12) (52 bits), u = (n + 0.5) * 2^-52, strictly
 *            inside (0, 1) and exact (2n + 1 has 53 bits); element e of a call comes from
 *            block counter + e / 2, words 2 (e % 2) and 2 (e % 2) + 1
 *   normal   the same Box-Muller in double on the block's two uniforms, a pair per block
 */
#include <mshadow/core/fastdiv.h>

#include "./abi_common.h"

using mshadow::FastDivU32;
using mshadow_abi::AfterLaunch;
using mshadow_abi::AsStream;

namespace {

const int kRandomBlock = 256;

struct Philox4 {
  uint32_t w[4];
};

/*! \brief one block of four 32-bit words */
__device__ __forceinline__ Philox4 Philox4x32_10(uint64_t seed, uint64_t subsequence,
                                                 uint64_t counter) {
  uint32_t c0 = static_cast<uint32_t>(counter), c1 = static_cast<uint32_t>(counter >> 32);
  uint32_t c2 = static_cast<uint32_t>(subsequence), c3 = static_cast<uint32_t>(subsequence >> 32);
  uint32_t k0 = static_cast<uint32_t>(seed), k1 = static_cast<uint32_t>(seed >> 32);
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    /* both halves of a 32 x 32 bit product from one instruction */
    uint64_t p0, p1;
    asm("v_mad_u64_u32 %0, vcc, %1, %2, 0" : "=v"(p0) : "v"(c0), "v"(0xD2511F53u) : "vcc");
    asm("v_mad_u64_u32 %0, vcc, %1, %2, 0" : "=v"(p1) : "v"(c2), "v"(0xCD9E8D57u) : "vcc");
    const uint32_t hi0 = static_cast<uint32_t>(p0 >> 32), lo0 = static_cast<uint32_t>(p0);
    const uint32_t hi1 = static_cast<uint32_t>(p1 >> 32), lo1 = static_cast<uint32_t>(p1);
    c0 = hi1 ^ c1 ^ k0;
    c1 = lo1;
    c2 = hi0 ^ c3 ^ k1;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  Philox4 out = {{c0, c1, c2, c3}};
  return out;
}

/*! \brief the top 23 bits of a word as a point strictly inside (0, 1): (n + 1/2) / 2^23 with
 *  n < 2^23, which is exact in float32 (2n + 1 has 24 bits), so the smallest value is 2^-24
 *  and the largest 1 - 2^-24; one bit more and n + 1/2 would round, up to 1 for the largest n */
__device__ __forceinline__ float UnitOpen(uint32_t x) {
  return (static_cast<float>(x >> 9) + 0.5f) * 1.1920928955078125e-07f;  // 2^-23
}

enum { kWords = 0, kUniform = 1, kNormal = 2 };

/*! \brief element e of the dense (rows, cols) view lands at row e / cols, column e % cols of
 *  a destination whose rows are `stride` elements apart; one thread per four elements */
/*! \brief PACKS: rows are whole aligned groups of four, so a thread's four values are
 *  neighbours in one row and leave as one 128-bit streaming store */
template <int KIND, bool PACKS>
__global__ void __launch_bounds__(kRandomBlock)
    RandomKernel(uint32_t *dst, uint32_t stride, uint32_t total, uint32_t cols, FastDivU32 div_cols,
                 uint64_t seed, uint64_t subsequence, uint64_t counter, float p0, float p1) {
  const uint32_t blocks = (total + 3u) / 4u;
  const uint32_t step = gridDim.x * kRandomBlock;
  for (uint32_t b = blockIdx.x * kRandomBlock + threadIdx.x; b < blocks; b += step) {
    const Philox4 r = Philox4x32_10(seed, subsequence, counter + b);
    uint32_t out[4];
    if (KIND == kWords) {
#pragma unroll
      for (int k = 0; k < 4; ++k) out[k] = r.w[k];
    } else if (KIND == kUniform) {
#pragma unroll
      for (int k = 0; k < 4; ++k) out[k] = __float_as_uint(UnitOpen(r.w[k]) * (p1 - p0) + p0);
    } else {
#pragma unroll
      for (int k = 0; k < 4; k += 2) {
        /* Box-Muller on the hardware's own functions: the arguments lie in [2^-24, 1), so
           none of the range handling of the library versions is needed. log2 -> ln by a
           factor; sine and cosine take their argument in revolutions */
        const float u = UnitOpen(r.w[k]), turn = UnitOpen(r.w[k + 1]);
        const float radius =
            __builtin_amdgcn_sqrtf(-1.3862943611198906f * __builtin_amdgcn_logf(u));  // -2 ln 2
        const float sn = __builtin_amdgcn_sinf(turn), cs = __builtin_amdgcn_cosf(turn);
        out[k] = __float_as_uint(p0 + radius * cs * p1);
        out[k + 1] = __float_as_uint(p0 + radius * sn * p1);
      }
    }
    if (PACKS) {
      const uint32_t e = b * 4u;
      const uint32_t y = div_cols.Div(e);
      typedef uint32_t V4 __attribute__((ext_vector_type(4)));
      V4 v;
      v.x = out[0], v.y = out[1], v.z = out[2], v.w = out[3];
      __builtin_nontemporal_store(
          v, reinterpret_cast<V4 *>(dst + static_cast<size_t>(y) * stride + (e - y * cols)));
      continue;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t e = b * 4u + k;
      if (e < total) {
        const uint32_t y = div_cols.Div(e);
        dst[static_cast<size_t>(y) * stride + (e - y * cols)] = out[k];
      }
    }
  }
}

/*! \brief 52 bits of two words as a point strictly inside (0, 1): (n + 1/2) / 2^52 */
__device__ __forceinline__ double UnitOpenDouble(uint32_t hi, uint32_t lo) {
  const uint64_t n = (static_cast<uint64_t>(hi) << 20) | (lo >> 12);
  return (static_cast<double>(n) + 0.5) * 2.220446049250313e-16;  // 2^-52
}

/*! \brief double values: a Philox block makes two of them; one thread per block. PAIRS: rows
 *  are whole aligned pairs, which leave as one 128-bit streaming store */
template <int KIND, bool PAIRS>
__global__ void __launch_bounds__(kRandomBlock)
    RandomDoubleKernel(double *dst, uint32_t stride, uint32_t total, uint32_t cols,
                       FastDivU32 div_cols, uint64_t seed, uint64_t subsequence, uint64_t counter,
                       double p0, double p1) {
  const uint32_t blocks = (total + 1u) / 2u;
  const uint32_t step = gridDim.x * kRandomBlock;
  for (uint32_t b = blockIdx.x * kRandomBlock + threadIdx.x; b < blocks; b += step) {
    const Philox4 r = Philox4x32_10(seed, subsequence, counter + b);
    const double u0 = UnitOpenDouble(r.w[0], r.w[1]), u1 = UnitOpenDouble(r.w[2], r.w[3]);
    double out[2];
    if (KIND == kUniform) {
      out[0] = u0 * (p1 - p0) + p0;
      out[1] = u1 * (p1 - p0) + p0;
    } else {
      const double radius = sqrt(-2.0 * log(u0));
      double sn, cs;
      sincospi(2.0 * u1, &sn, &cs);
      out[0] = p0 + radius * cs * p1;
      out[1] = p0 + radius * sn * p1;
    }
    if (PAIRS) {
      const uint32_t e = b * 2u;
      const uint32_t y = div_cols.Div(e);
      typedef double V2 __attribute__((ext_vector_type(2)));
      V2 v;
      v.x = out[0], v.y = out[1];
      __builtin_nontemporal_store(
          v, reinterpret_cast<V2 *>(dst + static_cast<size_t>(y) * stride + (e - y * cols)));
      continue;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const uint32_t e = b * 2u + k;
      if (e < total) {
        const uint32_t y = div_cols.Div(e);
        dst[static_cast<size_t>(y) * stride + (e - y * cols)] = out[k];
      }
    }
  }
}

template <int KIND>
int LaunchRandomDouble(double *dst, int dstride, int rows, int cols, uint64_t seed,
                       uint64_t subsequence, uint64_t counter, double p0, double p1, void *stream,
                       const char *what) {
  if (rows < 0 || cols < 0) return mshadow_abi::Fail(MSHADOW_HIP_ERR_ARGUMENT, std::string(what) + ": negative shape");
  if (rows == 0 || cols == 0) return MSHADOW_HIP_OK;
  if (dst == NULL) return mshadow_abi::Fail(MSHADOW_HIP_ERR_ARGUMENT, std::string(what) + ": NULL tensor");
  if (dstride < cols) return mshadow_abi::Fail(MSHADOW_HIP_ERR_ARGUMENT, std::string(what) + ": pitch smaller than the row");
  const uint64_t total = static_cast<uint64_t>(rows) * cols;
  if (total >= (1ull << 31)) return mshadow_abi::Fail(MSHADOW_HIP_ERR_ARGUMENT, std::string(what) + ": too many elements");
  uint64_t grid = ((total + 1) / 2 + kRandomBlock - 1) / kRandomBlock;
  if (grid > 16384) grid = 16384;
  const bool pairs = cols % 2 == 0 && dstride % 2 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0;
#define MSHADOW_RANDOM_LAUNCH(PAIRS)                                                              \
  hipLaunchKernelGGL((RandomDoubleKernel<KIND, PAIRS>), dim3(static_cast<unsigned>(grid)),        \
                     dim3(kRandomBlock), 0, AsStream(stream), dst, static_cast<uint32_t>(dstride), \
                     static_cast<uint32_t>(total), static_cast<uint32_t>(cols), FastDivU32(cols), \
                     seed, subsequence, counter, p0, p1)
  if (pairs) {
    MSHADOW_RANDOM_LAUNCH(true);
  } else {
    MSHADOW_RANDOM_LAUNCH(false);
  }
#undef MSHADOW_RANDOM_LAUNCH
  return AfterLaunch(what);
}

template <int KIND>
int LaunchRandom(void *dst, int dstride, int rows, int cols, uint64_t seed, uint64_t subsequence,
                 uint64_t counter, float p0, float p1, void *stream, const char *what) {
  if (rows < 0 || cols < 0) return mshadow_abi::Fail(MSHADOW_HIP_ERR_ARGUMENT, std::string(what) + ": negative shape");
  if (rows == 0 || cols == 0) return MSHADOW_HIP_OK;
  if (dst == NULL) return mshadow_abi::Fail(MSHADOW_HIP_ERR_ARGUMENT, std::string(what) + ": NULL tensor");
  if (dstride < cols) return mshadow_abi::Fail(MSHADOW_HIP_ERR_ARGUMENT, std::string(what) + ": pitch smaller than the row");
  const uint64_t total = static_cast<uint64_t>(rows) * cols;
  if (total >= (1ull << 31)) return mshadow_abi::Fail(MSHADOW_HIP_ERR_ARGUMENT, std::string(what) + ": too many elements");
  uint64_t grid = ((total + 3) / 4 + kRandomBlock - 1) / kRandomBlock;
  if (grid > 16384) grid = 16384;
  const bool packs = cols % 4 == 0 && dstride % 4 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0;
#define MSHADOW_RANDOM_LAUNCH(PACKS)                                                              \
  hipLaunchKernelGGL((RandomKernel<KIND, PACKS>), dim3(static_cast<unsigned>(grid)),              \
                     dim3(kRandomBlock), 0, AsStream(stream), static_cast<uint32_t *>(dst),       \
                     static_cast<uint32_t>(dstride), static_cast<uint32_t>(total),                \
                     static_cast<uint32_t>(cols), FastDivU32(cols), seed, subsequence, counter,   \
                     p0, p1)
  if (packs) {
    MSHADOW_RANDOM_LAUNCH(true);
  } else {
    MSHADOW_RANDOM_LAUNCH(false);
  }
#undef MSHADOW_RANDOM_LAUNCH
  return AfterLaunch(what);
}

}  // namespace

extern "C" {

int mshadow_hip_random_u32(uint32_t *dst, size_t n, uint64_t seed, uint64_t subsequence,
                           uint64_t counter, void *stream) {
  ABI_REQUIRE(n < (1ull << 31), "too many elements");
  return LaunchRandom<kWords>(dst, static_cast<int>(n), 1, static_cast<int>(n), seed, subsequence,
                              counter, 0.0f, 0.0f, stream, "random_u32");
}

int mshadow_hip_random_uniform_f32(float *dst, int dstride, int rows, int cols, uint64_t seed,
                                   uint64_t subsequence, uint64_t counter, float a, float b,
                                   void *stream) {
  return LaunchRandom<kUniform>(dst, dstride, rows, cols, seed, subsequence, counter, a, b, stream,
                                "random_uniform");
}

int mshadow_hip_random_normal_f32(float *dst, int dstride, int rows, int cols, uint64_t seed,
                                  uint64_t subsequence, uint64_t counter, float mu, float sigma,
                                  void *stream) {
  return LaunchRandom<kNormal>(dst, dstride, rows, cols, seed, subsequence, counter, mu, sigma,
                               stream, "random_normal");
}

int mshadow_hip_random_uniform_f64(double *dst, int dstride, int rows, int cols, uint64_t seed,
                                   uint64_t subsequence, uint64_t counter, double a, double b,
                                   void *stream) {
  return LaunchRandomDouble<kUniform>(dst, dstride, rows, cols, seed, subsequence, counter, a, b,
                                      stream, "random_uniform_f64");
}

int mshadow_hip_random_normal_f64(double *dst, int dstride, int rows, int cols, uint64_t seed,
                                  uint64_t subsequence, uint64_t counter, double mu, double sigma,
                                  void *stream) {
  return LaunchRandomDouble<kNormal>(dst, dstride, rows, cols, seed, subsequence, counter, mu, sigma,
                                     stream, "random_normal_f64");
}

}  // extern "C"
