/*
 * Wave64 building blocks shared by the gfx950 kernels (device code, hipcc only).
 *
 * A gfx950 wavefront has 64 lanes; cross-lane data movement below uses the wave
 * shuffle / broadcast instructions, never a 32-lane assumption. The reference's
 * shared-memory tree with a warp-synchronous tail (mshadow/cuda/reduce.cuh:42-116)
 * is what these replace.
 */
#ifndef MSHADOW_HIP_KERNELS_COMMON_H_
#define MSHADOW_HIP_KERNELS_COMMON_H_

#if !defined(__HIPCC__)
#error "mshadow/hip/kernels/*.h hold device code: compile this translation unit with hipcc"
#endif

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../base.h"

namespace mshadow {
namespace hip {

const int kWave = 64;

__device__ __forceinline__ int LaneId() { return threadIdx.x & (kWave - 1); }
__device__ __forceinline__ int WaveId() { return threadIdx.x >> 6; }

/*! \brief value of `v` in lane `lane` (same lane for the whole wave), as a scalar */
__device__ __forceinline__ uint32_t ReadLaneU32(uint32_t v, int lane) {
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v),
                                                         __builtin_amdgcn_readfirstlane(lane)));
}
__device__ __forceinline__ float ReadLaneF32(float v, int lane) {
  return __uint_as_float(ReadLaneU32(__float_as_uint(v), lane));
}

/*! \brief max over the 64 lanes with operator< semantics; result in every lane */
__device__ __forceinline__ float WaveMaxF32(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off, kWave);
    v = (v < o) ? o : v;
  }
  return v;
}
/*! \brief sum over the 64 lanes; result in every lane */
__device__ __forceinline__ uint32_t WaveSumU32(uint32_t v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
/*! \brief inclusive prefix sum over lanes 0..63 */
__device__ __forceinline__ uint32_t WaveInclusiveScanU32(uint32_t v) {
  const int lane = LaneId();
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t o = __shfl_up(v, off, kWave);
    if (lane >= off) v += o;
  }
  return v;
}

/*! \brief does Saver::Save read the old destination value? (only plain assignment
 *  does not; savers the library does not know are assumed to) */
template <typename Saver>
struct SaverReadsDst {
  static const bool value = true;
};
template <>
struct SaverReadsDst<sv::saveto> {
  static const bool value = false;
};

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_COMMON_H_
