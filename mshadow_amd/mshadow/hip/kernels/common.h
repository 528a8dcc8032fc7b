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
/*! \brief inclusive prefix maximum of unsigned integers over lanes 0..63 (one DPP
 *  instruction per step, each behind the idle cycles the hardware asks for) */
__device__ __forceinline__ uint32_t WaveInclusiveScanMaxU32(uint32_t v) {
  asm volatile(
      "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
      "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:2 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
      "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:4 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
      "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:8 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
      "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1"
      : "+v"(v));
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
#define MSHADOW_DPP_QUAD_PERM(a, b, c, d) ((a) | ((b) << 2) | ((c) << 4) | ((d) << 6))
#define MSHADOW_DPP_ROW_ROR(n) (0x120 + (n))   // lane i reads lane (i + n) % 16 of its row

/*! \brief value of `v` in the lane paired with this one at distance D: lane ^ D for
 *  D = 1, 2, 8, 16, 32 and (lane + 4) % 16 within the row for D = 4 - in every case a lane
 *  whose bit log2(D) is the opposite of this lane's, which is all WaveReduceMany needs */
template <int D>
__device__ __forceinline__ uint32_t PairedLaneU32(uint32_t u) {
  if (D == 1) return DppU32<MSHADOW_DPP_QUAD_PERM(1, 0, 3, 2), 0xf>(u, u);
  if (D == 2) return DppU32<MSHADOW_DPP_QUAD_PERM(2, 3, 0, 1), 0xf>(u, u);
  if (D == 4) return DppU32<MSHADOW_DPP_ROW_ROR(4), 0xf>(u, u);
  if (D == 8) return DppU32<MSHADOW_DPP_ROW_ROR(8), 0xf>(u, u);
  return static_cast<uint32_t>(__shfl_xor(static_cast<int>(u), D));
}
template <int D>
__device__ __forceinline__ float PairedLaneF32(float v) {
  return __uint_as_float(PairedLaneU32<D>(__float_as_uint(v)));
}
template <int D>
__device__ __forceinline__ uint32_t PairedLane(uint32_t v) { return PairedLaneU32<D>(v); }
template <int D>
__device__ __forceinline__ float PairedLane(float v) { return PairedLaneF32<D>(v); }

/*! \brief the combining steps WaveReduceMany can be asked for */
struct WaveOpSum {
  template <typename T>
  static __device__ __forceinline__ T Do(T a, T b) { return a + b; }
};
struct WaveOpMax {  // operator< semantics, like red::maximum
  template <typename T>
  static __device__ __forceinline__ T Do(T a, T b) { return (a < b) ? b : a; }
  /* floats: one instruction (a NaN operand is ignored) instead of a compare and a select */
  static __device__ __forceinline__ float Do(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
  }
};

/*! \brief M reductions over the wave at once (M a power of two up to 32): returns, in lane
 *  l, the reduction over all 64 lanes of a[l % M]. Each of the first log2(M) steps halves
 *  the number of values a lane carries (it keeps the values whose index has this lane's bit
 *  and hands the others to its paired lane), so the whole thing costs about M + 2 * 6
 *  combining steps instead of 6 * M. `a` is clobbered. Sums are exact on integers and on
 *  integer-valued floats below 2^24; on other floats the order of additions differs from
 *  a scan. */
template <typename Op, typename T, int M, int S = 0>
struct WaveReduceManyStep {
  static __device__ __forceinline__ void Run(T (&a)[M]) {
    const bool bit = (threadIdx.x >> S) & 1;
    const int CNT = M >> (S + 1);
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const T keep = bit ? a[2 * i + 1] : a[2 * i];
      const T send = bit ? a[2 * i] : a[2 * i + 1];
      a[i] = Op::Do(keep, PairedLane<(1 << S)>(send));
    }
    WaveReduceManyStep<Op, T, M, ((2 << S) < M) ? S + 1 : 64>::Run(a);
  }
};
template <typename Op, typename T, int M>
struct WaveReduceManyStep<Op, T, M, 64> {
  static __device__ __forceinline__ void Run(T (&)[M]) {}
};
template <typename Op, typename T, int M, int D>
struct WaveReduceRest {
  static __device__ __forceinline__ T Run(T r) {
    return WaveReduceRest<Op, T, M, D * 2>::Run(Op::Do(r, PairedLane<D>(r)));
  }
};
template <typename Op, typename T, int M>
struct WaveReduceRest<Op, T, M, 64> {
  static __device__ __forceinline__ T Run(T r) { return r; }
};
template <typename Op, typename T, int M>
__device__ __forceinline__ T WaveReduceMany(T (&a)[M]) {
  if (M > 1) WaveReduceManyStep<Op, T, M, (M > 1 ? 0 : 64)>::Run(a);
  return WaveReduceRest<Op, T, M, M>::Run(a[0]);
}
template <int M>
__device__ __forceinline__ float WaveSumMany(float (&a)[M]) {
  return WaveReduceMany<WaveOpSum, float, M>(a);
}

/*! \brief inclusive prefix maximum over lanes 0..63 of non-negative floats (a lane with
 *  no source in a step sees 0, which is the identity for them; NaN operands are ignored).
 *  One DPP instruction per step; the idle cycles in front of each are what the hardware
 *  asks for between writing a register and reading it through DPP. */
__device__ __forceinline__ float WaveInclusiveScanMaxF32(float v) {
  asm volatile(
      "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
      "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_shr:2 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
      "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_shr:4 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
      "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_shr:8 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
      "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1"
      : "+v"(v));
  return v;
}

/* Several scans at once: the steps of the scans are interleaved, so that the idle cycles the
   hardware asks for between writing a register and reading it through DPP are filled by
   the other scans' steps instead of waiting, and the chains of dependent steps overlap. */
#define MSHADOW_SCAN_CTRLS(X)                                  \
  X("row_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1")       \
  X("row_shr:2 row_mask:0xf bank_mask:0xf bound_ctrl:1")       \
  X("row_shr:4 row_mask:0xf bank_mask:0xf bound_ctrl:1")       \
  X("row_shr:8 row_mask:0xf bank_mask:0xf bound_ctrl:1")       \
  X("row_bcast:15 row_mask:0xa bank_mask:0xf")                 \
  X("row_bcast:31 row_mask:0xc bank_mask:0xf")
/*! \brief inclusive prefix sum of *sum and inclusive prefix maximum of *mx (non-negative
 *  floats) over lanes 0..63 */
__device__ __forceinline__ void WaveScanSumAndMaxF32(float *sum, float *mx) {
#define MSHADOW_STEP(CTRL)                      \
  "v_add_f32_dpp %0, %0, %0 " CTRL "\n\t"       \
  "v_max_f32_dpp %1, %1, %1 " CTRL "\n\t"       \
  "s_nop 0\n\t"
  asm volatile("s_nop 1\n\t" MSHADOW_SCAN_CTRLS(MSHADOW_STEP) "s_nop 0" : "+v"(*sum), "+v"(*mx));
#undef MSHADOW_STEP
}
/*! \brief inclusive prefix sums of *a, *b and *c (unsigned) over lanes 0..63 */
__device__ __forceinline__ void WaveScanSum3U32(uint32_t *a, uint32_t *b, uint32_t *c) {
#define MSHADOW_STEP(CTRL)                      \
  "v_add_u32_dpp %0, %0, %0 " CTRL "\n\t"       \
  "v_add_u32_dpp %1, %1, %1 " CTRL "\n\t"       \
  "v_add_u32_dpp %2, %2, %2 " CTRL "\n\t"
  asm volatile("s_nop 1\n\t" MSHADOW_SCAN_CTRLS(MSHADOW_STEP) "s_nop 1"
               : "+v"(*a), "+v"(*b), "+v"(*c));
#undef MSHADOW_STEP
}
/*! \brief number of set bits of `mask` below this lane */
__device__ __forceinline__ uint32_t LanesBelow(unsigned long long mask) {
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
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

/*! \brief which piece of the work a workgroup takes. Workgroups are dealt to the 8 XCDs
 *  round-robin, and each XCD has its own L2: handing XCD k the k-th contiguous eighth of
 *  the pieces (when the count divides evenly) keeps neighbouring pieces - which share
 *  cache lines, halos or, for windowed expressions, whole operands - behind one L2. */
__device__ __forceinline__ uint32_t StripOfBlock(uint32_t block, uint32_t nblocks) {
  const uint32_t kXcd = 8;
  if (nblocks % kXcd != 0) return block;
  return (block % kXcd) * (nblocks / kXcd) + block / kXcd;
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_COMMON_H_
