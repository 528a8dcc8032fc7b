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

/* DPP (data-parallel primitive) controls of the GFX9 family: a VALU operand is taken
   from another lane of the same wave without going through LDS. A row is 16 lanes. */
#define MSHADOW_DPP_ROW_SHR(n) (0x110 + (n))  // lane i reads lane i-n of its row
#define MSHADOW_DPP_ROW_BCAST15 0x142          // lane 15 of each row -> every lane of the next row
#define MSHADOW_DPP_ROW_BCAST31 0x143          // lane 31 -> every lane of rows 2 and 3

/*! \brief src of the DPP-selected lane; lanes that have no source (or are masked off by
 *  row_mask) receive `old` */
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t DppU32(uint32_t old, uint32_t src) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(
      static_cast<int>(old), static_cast<int>(src), CTRL, ROW_MASK, 0xf, false));
}

/*! \brief inclusive prefix sum over lanes 0..63: Hillis-Steele inside each 16-lane row
 *  (shifts 1, 2, 4, 8), then the row totals carried across rows. Six VALU steps. */
__device__ __forceinline__ uint32_t WaveInclusiveScanU32(uint32_t v) {
  v += DppU32<MSHADOW_DPP_ROW_SHR(1), 0xf>(0u, v);
  v += DppU32<MSHADOW_DPP_ROW_SHR(2), 0xf>(0u, v);
  v += DppU32<MSHADOW_DPP_ROW_SHR(4), 0xf>(0u, v);
  v += DppU32<MSHADOW_DPP_ROW_SHR(8), 0xf>(0u, v);
  v += DppU32<MSHADOW_DPP_ROW_BCAST15, 0xa>(0u, v);
  v += DppU32<MSHADOW_DPP_ROW_BCAST31, 0xc>(0u, v);
  return v;
}
/*! \brief the same for floats (used on integer-valued floats, where it is exact below 2^24) */
__device__ __forceinline__ float WaveInclusiveScanF32(float v) {
#define MSHADOW_FSCAN_STEP(CTRL, MASK) \
  v += __uint_as_float(DppU32<CTRL, MASK>(0u, __float_as_uint(v)));
  MSHADOW_FSCAN_STEP(MSHADOW_DPP_ROW_SHR(1), 0xf)
  MSHADOW_FSCAN_STEP(MSHADOW_DPP_ROW_SHR(2), 0xf)
  MSHADOW_FSCAN_STEP(MSHADOW_DPP_ROW_SHR(4), 0xf)
  MSHADOW_FSCAN_STEP(MSHADOW_DPP_ROW_SHR(8), 0xf)
  MSHADOW_FSCAN_STEP(MSHADOW_DPP_ROW_BCAST15, 0xa)
  MSHADOW_FSCAN_STEP(MSHADOW_DPP_ROW_BCAST31, 0xc)
#undef MSHADOW_FSCAN_STEP
  return v;
}
/*! \brief sum over the 64 lanes; result in every lane (as a scalar) */
__device__ __forceinline__ uint32_t WaveSumU32(uint32_t v) {
  return ReadLaneU32(WaveInclusiveScanU32(v), kWave - 1);
}
/*! \brief max over the 64 lanes with operator< semantics; result in every lane */
__device__ __forceinline__ float WaveMaxF32(float v) {
#define MSHADOW_MAX_STEP(CTRL, MASK)                                                      \
  {                                                                                       \
    const float o = __uint_as_float(DppU32<CTRL, MASK>(__float_as_uint(v), __float_as_uint(v))); \
    v = (v < o) ? o : v;                                                                  \
  }
  MSHADOW_MAX_STEP(MSHADOW_DPP_ROW_SHR(1), 0xf)
  MSHADOW_MAX_STEP(MSHADOW_DPP_ROW_SHR(2), 0xf)
  MSHADOW_MAX_STEP(MSHADOW_DPP_ROW_SHR(4), 0xf)
  MSHADOW_MAX_STEP(MSHADOW_DPP_ROW_SHR(8), 0xf)
  MSHADOW_MAX_STEP(MSHADOW_DPP_ROW_BCAST15, 0xa)
  MSHADOW_MAX_STEP(MSHADOW_DPP_ROW_BCAST31, 0xc)
#undef MSHADOW_MAX_STEP
  return ReadLaneF32(v, kWave - 1);  // lane 63 holds the running maximum of all lanes
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
