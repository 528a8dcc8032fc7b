/*
 * SortByKey for key and value types the library's 32-bit sort does not take directly
 * (mshadow/tensor_gpu-inl.h:231-235: any key type with an order, any value type; the
 * reference hands both to thrust::stable_sort_by_key).
 *
 * The library sorts (32-bit key, 32-bit value) pairs stably. A key of another width is sorted
 * through a permutation: the keys are mapped to unsigned words whose order is the keys' order,
 * the permutation 0..n-1 is sorted by the low word and then, stably, by the high word (64-bit
 * keys; narrower keys need one pass on a widened copy), and keys and values are finally
 * gathered through the permutation. Stability of each pass makes the whole sort stable, in
 * both directions. Keys that compare equal must map to the same word: -0.0 is mapped as +0.0.
 */
#ifndef MSHADOW_HIP_KERNELS_SORT_ANY_H_
#define MSHADOW_HIP_KERNELS_SORT_ANY_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mshadow {
namespace hip {

const int kSortAnyBlock = 256;

/*! \brief keys as unsigned 64-bit numbers of the same order */
__device__ __forceinline__ uint64_t OrderedBits(double k) {
  if (k == 0.0) k = 0.0;  // -0.0 and +0.0 are one key
  const uint64_t b = static_cast<uint64_t>(__double_as_longlong(k));
  return (b >> 63) ? ~b : (b | 0x8000000000000000ull);
}
__device__ __forceinline__ uint64_t OrderedBits(float k) {
  if (k == 0.0f) k = 0.0f;
  const uint32_t b = __float_as_uint(k);
  return (b >> 31) ? static_cast<uint32_t>(~b) : (b | 0x80000000u);
}
__device__ __forceinline__ uint64_t OrderedBits(int64_t k) {
  return static_cast<uint64_t>(k) ^ 0x8000000000000000ull;
}
__device__ __forceinline__ uint64_t OrderedBits(uint64_t k) { return k; }
__device__ __forceinline__ uint64_t OrderedBits(long long k) {
  return static_cast<uint64_t>(k) ^ 0x8000000000000000ull;
}
__device__ __forceinline__ uint64_t OrderedBits(unsigned long long k) { return k; }
__device__ __forceinline__ uint64_t OrderedBits(int32_t k) { return static_cast<uint32_t>(k) ^ 0x80000000u; }
__device__ __forceinline__ uint64_t OrderedBits(uint32_t k) { return k; }
__device__ __forceinline__ uint64_t OrderedBits(int16_t k) { return static_cast<uint32_t>(static_cast<int32_t>(k)) ^ 0x80000000u; }
__device__ __forceinline__ uint64_t OrderedBits(uint16_t k) { return k; }
__device__ __forceinline__ uint64_t OrderedBits(int8_t k) { return static_cast<uint32_t>(static_cast<int32_t>(k)) ^ 0x80000000u; }
__device__ __forceinline__ uint64_t OrderedBits(uint8_t k) { return k; }
__device__ __forceinline__ uint64_t OrderedBits(char k) { return OrderedBits(static_cast<int8_t>(k)); }
__device__ __forceinline__ uint64_t OrderedBits(bool k) { return k ? 1u : 0u; }

/*! \brief word[i] = the HIGH or low 32 bits of the ordered form of keys[perm[i]] (perm NULL:
 *  of keys[i], and perm_out[i] = i is written as the starting permutation) */
template <typename KDType, bool HIGH>
__global__ void __launch_bounds__(kSortAnyBlock)
    SortKeyWordKernel(uint32_t *word, uint32_t *perm_out, const KDType *keys, const uint32_t *perm,
                      uint32_t n) {
  for (uint32_t i = blockIdx.x * kSortAnyBlock + threadIdx.x; i < n; i += gridDim.x * kSortAnyBlock) {
    const uint32_t from = perm != NULL ? perm[i] : i;
    const uint64_t b = OrderedBits(keys[from]);
    word[i] = HIGH ? static_cast<uint32_t>(b >> 32) : static_cast<uint32_t>(b);
    if (perm == NULL) perm_out[i] = i;
  }
}

/*! \brief dst[i] = src[perm[i]] */
template <typename T>
__global__ void __launch_bounds__(kSortAnyBlock)
    SortGatherKernel(T *dst, const T *src, const uint32_t *perm, uint32_t n) {
  for (uint32_t i = blockIdx.x * kSortAnyBlock + threadIdx.x; i < n; i += gridDim.x * kSortAnyBlock) {
    dst[i] = src[perm[i]];
  }
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_SORT_ANY_H_
