/*
 * Softmax / SoftmaxGrad for element types other than float (half_t, double), written in the
 * element type's own arithmetic so that every intermediate rounds where the CPU path rounds
 * (mshadow/tensor_cpu-inl.h:270-302): the difference x - max, the exponential stored into
 * dst, the running sum after every add and the final quotient are all values of DType.
 * For half_t that matters: a sum kept in 16 bits stops growing once its ulp exceeds twice the
 * terms (4096 equal logits give 1/2048 each, not 1/4096), and only the left-to-right order
 * reproduces it.
 *
 * One wave per row, four rows per workgroup. The maximum is a wave reduction (exact in any
 * order). The row then passes in tiles of 64 lanes x kAnyTile consecutive terms: every lane
 * computes its terms, stores them to dst and parks them in LDS; lane 0 adds the tile to the
 * running sum term by term (the dependent chain is the cost of the kernel: 32 rows are
 * resident per CU so that the chains of different rows overlap). A last pass divides; each
 * lane reads back only what it stored itself, so in-place calls (dst == src) are safe.
 *
 * The float versions are the fixed-function kernels of the library (csrc/softmax_kernels.h).
 */
#ifndef MSHADOW_HIP_KERNELS_SOFTMAX_ANY_H_
#define MSHADOW_HIP_KERNELS_SOFTMAX_ANY_H_

#include "../../half.h"
#include "./common.h"

namespace mshadow {
namespace hip {

const int kAnyBlock = 256;
const int kAnyRowsPerBlock = kAnyBlock / kWave;
/*! \brief consecutive terms of one lane in a tile */
const int kAnyTile = 8;

/*! \brief what std::exp(DType) resolves to on the host: the float function for half_t
 *  (through its conversion to float) and float, the double function for double */
__device__ __forceinline__ float SoftmaxExp(half::half_t v) { return expf(static_cast<float>(v)); }
__device__ __forceinline__ float SoftmaxExp(float v) { return expf(v); }
__device__ __forceinline__ double SoftmaxExp(double v) { return exp(v); }

/*! \brief the type comparisons of DType are made in (exact widening) */
template <typename DType>
struct WideOf { typedef float Type; };
template <>
struct WideOf<double> { typedef double Type; };

/*! \brief static_cast<int>(label) as the host makes it: half_t goes through float */
__device__ __forceinline__ int LabelIndex(half::half_t v) { return static_cast<int>(static_cast<float>(v)); }
__device__ __forceinline__ int LabelIndex(float v) { return static_cast<int>(v); }
__device__ __forceinline__ int LabelIndex(double v) { return static_cast<int>(v); }

__device__ __forceinline__ float WaveShuffleXor(float v, int mask) { return __shfl_xor(v, mask); }
__device__ __forceinline__ double WaveShuffleXor(double v, int mask) { return __shfl_xor(v, mask); }

template <typename DType>
__global__ void __launch_bounds__(kAnyBlock)
    SoftmaxAnyKernel(DType *dst, uint32_t dstride, const DType *src, uint32_t sstride,
                     uint32_t rows, uint32_t cols) {
  typedef typename WideOf<DType>::Type Wide;
  const int kTileElems = kWave * kAnyTile;
  __shared__ DType tile[kAnyRowsPerBlock][kTileElems];
  __shared__ DType sums[kAnyRowsPerBlock];
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t row = blockIdx.x * kAnyRowsPerBlock + wave;
  /* a wave without a row runs along (the barriers are the workgroup's) and touches nothing */
  const bool live = row < rows;
  const DType *e = src + static_cast<size_t>(live ? row : 0) * sstride;
  DType *o = dst + static_cast<size_t>(live ? row : 0) * dstride;

  /* maximum: `if (mmax < e[x]) mmax = e[x]` from e[0] on, which is the largest value */
  Wide m = static_cast<Wide>(e[0]);
  if (live) {
    for (uint32_t x = lane; x < cols; x += kWave) {
      const Wide v = static_cast<Wide>(e[x]);
      m = (m < v) ? v : m;
    }
  }
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const Wide other = WaveShuffleXor(m, d);
    m = (m < other) ? other : m;
  }
  const DType mmax = static_cast<DType>(m);  // exact: m is one of the row's values

  DType sum = DType(0.0f);
  for (uint32_t x0 = 0; x0 < cols; x0 += kTileElems) {
    if (live) {
#pragma unroll
      for (int i = 0; i < kAnyTile; ++i) {
        const uint32_t x = x0 + lane * kAnyTile + i;
        if (x < cols) {
          const DType t = DType(SoftmaxExp(e[x] - mmax));
          o[x] = t;
          tile[wave][lane * kAnyTile + i] = t;
        }
      }
    }
    __syncthreads();
    if (live && lane == 0) {
      const uint32_t n = cols - x0 < static_cast<uint32_t>(kTileElems) ? cols - x0 : kTileElems;
      uint32_t j = 0;
      for (; j + 8 <= n; j += 8) {
        DType t[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] = tile[wave][j + i];
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += t[i];
      }
      for (; j < n; ++j) sum += tile[wave][j];
    }
    __syncthreads();
  }
  if (lane == 0) sums[wave] = sum;
  __syncthreads();
  sum = sums[wave];

  if (live) {
    for (uint32_t x0 = 0; x0 < cols; x0 += kTileElems) {
#pragma unroll
      for (int i = 0; i < kAnyTile; ++i) {
        const uint32_t x = x0 + lane * kAnyTile + i;
        if (x < cols) {
          DType v = o[x];
          v /= sum;
          o[x] = v;
        }
      }
    }
  }
}

/*! \brief dst = src with 1 subtracted at column static_cast<int>(label[row]); a label
 *  outside the row leaves a copy. blockIdx.x = row, blockIdx.y = stretch of columns. */
template <typename DType>
__global__ void __launch_bounds__(kAnyBlock)
    SoftmaxGradAnyKernel(DType *dst, uint32_t dstride, const DType *src, uint32_t sstride,
                         const DType *label, uint32_t cols) {
  const uint32_t row = blockIdx.x;
  const int k = LabelIndex(label[row]);
  const DType *s = src + static_cast<size_t>(row) * sstride;
  DType *o = dst + static_cast<size_t>(row) * dstride;
  for (uint32_t x = blockIdx.y * kAnyBlock + threadIdx.x; x < cols; x += gridDim.y * kAnyBlock) {
    DType v = s[x];
    if (static_cast<int>(x) == k) v = v - 1.0f;
    o[x] = v;
  }
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_SOFTMAX_ANY_H_
