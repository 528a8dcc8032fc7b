/*
 * Reduce-to-1D of a plain float tensor with the loads delivered straight into LDS.
 *
 * Same order of operations as the kernels in reduce.h (one serial chain per output, see
 * there for why), different plumbing. When the source is a tensor in memory - not an
 * expression that has to be evaluated in registers - the loader waves use the
 * global-load-to-LDS instruction of gfx950: the data never passes through VGPRs, so the
 * depth of the pipeline is limited by LDS (a ring of 128 KB: up to six stages = 96 KB
 * per CU in flight) instead of by registers and by what the compiler can prove
 * about loop-carried loads. Roles are fixed per wave:
 *   waves 1..8  issue the loads of stage i, wait (by count) for their own loads of
 *               an earlier stage to have landed, and meet the barrier; they never read LDS,
 *               fetch nothing past the last stage and exit with no load outstanding;
 *   wave 0      after the barrier folds that stage from its slot with 128-bit LDS reads,
 *               one dependent add per element; it never touches global memory.
 * A slot is refilled two barriers after the chain has finished with it.
 *
 * The load instruction places lane l's dword at (wave base + 4 l) in LDS, so the layout
 * of a slot is chosen per kernel such that the lanes of one instruction fetch full
 * 64-byte runs of global memory AND a chain lane finds four consecutive operands in one
 * 16-byte LDS word.
 *
 * The barrier here is the bare instruction: the usual workgroup fence in front of it
 * would wait for every outstanding load, which is exactly what the ring avoids. Ordering
 * is by construction: a loader's wait-by-count precedes its barrier, and the chain's LDS
 * reads have returned (their sums depend on them) before it reaches the next barrier.
 */
#ifndef MSHADOW_HIP_KERNELS_REDUCE_DMA_H_
#define MSHADOW_HIP_KERNELS_REDUCE_DMA_H_

#include "../../core/fastdiv.h"
#include "./common.h"
#include "./reduce.h"

namespace mshadow {
namespace hip {

/*! \brief loader waves per workgroup (one more wave runs the chains) */
const int kDmaLoaders = 8;
const int kDmaThreads = (kDmaLoaders + 1) * kWave;
/*! \brief LDS ring of SLOTS slots of ELEMS floats each (128 KB in all): SLOTS - 2 stages
 *  are in flight. KeepHighDim is bound by HBM and takes many small stages (deep queue);
 *  KeepLowest is bound by its chain of dependent adds and takes few large ones, so that
 *  the LDS latency at the start of a stage is paid less often. */
template <int SLOTS_, int ELEMS_>
struct DmaRing {
  static const int kSlots = SLOTS_;
  static const int kElems = ELEMS_;
  static const int kAhead = SLOTS_ - 2;
  /*! \brief load instructions per loader wave per stage (64 dwords each) */
  static const int kPerWave = ELEMS_ / kWave / kDmaLoaders;
  static_assert(kAhead * kPerWave < 64, "the wait-by-count immediate has 6 bits");
};
typedef DmaRing<4, 8192> LowestRing;
typedef DmaRing<8, 4096> HighDimRing;

/*! \brief cache policy of the loads: non-temporal (the data passes through once; measured
 *  38 us against 43 us for the (64,256,56,56) reduction) */
const int kDmaCachePolicy = 2;
/*! \brief lane l of the wave fetches the 4 bytes at gsrc_of_lane into the l-th dword behind
 *  lds_wave_base */
__device__ __forceinline__ void LoadDwordToLds(const void *gsrc_of_lane, void *lds_wave_base) {
  __builtin_amdgcn_global_load_lds(
      (const __attribute__((address_space(1))) void *)gsrc_of_lane,
      (__attribute__((address_space(3))) void *)lds_wave_base, 4, 0, kDmaCachePolicy);
}
/*! \brief all but the newest kAhead stages of this wave's loads have landed */
template <typename Ring>
__device__ __forceinline__ void WaitStageLanded() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(Ring::kAhead * Ring::kPerWave) : "memory");
}
/*! \brief every load of this wave has landed (used once the last stage has been issued:
 *  nothing is fetched past the end, and no load is outstanding when the wave exits and
 *  the workgroup's LDS is handed to the next one) */
__device__ __forceinline__ void WaitAllLanded() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void BareBarrier() { asm volatile("s_barrier" ::: "memory"); }

/* ------------------------------------------------------------------ KeepLowest
 * 16 columns per workgroup. A stage is 512 rows; one load instruction covers a group of
 * four rows: lane l fetches row 4 g + (l & 3), column l >> 2, so the slot holds
 * [group][column][row & 3] and a chain lane reads rows 4g..4g+3 of its column as one
 * 128-bit word, 64 floats from the next group. */
template <typename Saver, typename Reducer>
__global__ void __launch_bounds__(kDmaThreads)
    ReduceKeepLowestDmaKernel(float *dst, const float *src, uint32_t stride, uint32_t rows,
                              uint32_t cols, float scale) {
  typedef LowestRing Ring;
  const int kDmaSlots = Ring::kSlots, kDmaAhead = Ring::kAhead, kDmaPerWave = Ring::kPerWave;
  const int CW = kLowestCols;
  const int TR = Ring::kElems / CW;
  __shared__ MSHADOW_ALIGNED(16) float ring[Ring::kSlots][Ring::kElems];

  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t x0 = StripOfBlock(blockIdx.x, gridDim.x) * CW;
  const uint32_t nstage = (rows + TR - 1) / TR;
  const uint32_t nstep = nstage == 0 ? 0 : nstage + kDmaAhead;

  if (wave != 0) {
    const uint32_t lw = wave - 1;
    const uint32_t r = lane & 3;
    /* out-of-range columns and rows re-read the last valid one: never consumed */
    const uint32_t xc = (x0 + (lane >> 2) < cols) ? x0 + (lane >> 2) : cols - 1;
    const float *colp = src + xc;
    for (uint32_t i = 0; i < nstep; ++i) {
      if (i < nstage) {
        float *slot = ring[i % kDmaSlots];
#pragma unroll
        for (int q = 0; q < kDmaPerWave; ++q) {
          const uint32_t g = q * kDmaLoaders + lw;
          uint32_t row = i * TR + g * 4 + r;
          row = row < rows ? row : rows - 1;
          LoadDwordToLds(colp + static_cast<size_t>(row) * stride, slot + g * kWave);
        }
        WaitStageLanded<Ring>();
      } else {
        WaitAllLanded();
      }
      BareBarrier();
    }
  } else {
    const bool chain_lane = lane < static_cast<uint32_t>(CW) && x0 + lane < cols;
    float res = 0.0f;
    for (uint32_t i = 0; i < nstep; ++i) {
      BareBarrier();
      if (i >= static_cast<uint32_t>(kDmaAhead) && chain_lane) {
        const uint32_t st = i - kDmaAhead;
        const uint32_t row0 = st * TR;
        const float *mine = ring[st % kDmaSlots] + lane * 4;
        const int count = (rows - row0 < (uint32_t)TR) ? static_cast<int>(rows - row0) : TR;
        int begin = 0;
        if (st == 0) {  // the reference starts from src(0, x), not from an initial value
          res = mine[0];
          begin = 1;
        }
        ChainFold<Reducer, kWave>(res, mine, begin, count);
      }
    }
    if (chain_lane) Saver::template Save<float>(dst[x0 + lane], res * scale);
  }
}

/* ------------------------------------------------------------------ KeepHighDim
 * shape viewed as (n_out, n_keep, n_y, n_x); one workgroup per kept index c; SEGS inner
 * segments (n values) side by side in a slot, TL = 4096 / SEGS elements of each per
 * stage, one chain lane per segment. One load instruction fetches 64 consecutive
 * elements of one segment into their place in the slot. */
/* The element type is float or a 16-bit type: a load moves a dword per lane, i.e. one float or
 * two neighbouring 16-bit elements, which must then lie in one row of the source (n_x and the
 * pitch even, the base 4-byte aligned: the launcher's business). */
template <typename Saver, typename Reducer, typename DType, int SEGS>
__global__ void __launch_bounds__(kDmaThreads)
    ReduceKeepHighDimDmaKernel(DType *dst, const DType *src, uint32_t stride, uint32_t n_out,
                               uint32_t n_keep, uint32_t n_y, uint32_t n_x, FastDivU32 div_x,
                               DType scale) {
  typedef HighDimRing Ring;
  const int kDmaSlots = Ring::kSlots, kDmaAhead = Ring::kAhead, kDmaPerWave = Ring::kPerWave;
  const int EPD = 4 / sizeof(DType);       // elements per dword
  const int TL = Ring::kElems * EPD / SEGS;
  const int LD = TL + 16 / sizeof(DType);  // chain lanes read words LD elements apart: no bank conflicts
  static_assert(sizeof(DType) == 4 || sizeof(DType) == 2, "a dword holds one or two elements");
  static_assert(TL % (kWave * EPD) == 0, "an instruction stays inside one segment");
  __shared__ MSHADOW_ALIGNED(16) DType ring[Ring::kSlots][SEGS * LD];

  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t c = blockIdx.x;
  const uint32_t seg_len = n_y * n_x;
  const uint32_t stages_per_group = (seg_len + TL - 1) / TL;
  const uint32_t groups = (n_out + SEGS - 1) / SEGS;
  const uint32_t nstage = groups * stages_per_group;
  const uint32_t nstep = nstage == 0 ? 0 : nstage + kDmaAhead;

  if (wave != 0) {
    const uint32_t lw = wave - 1;
    uint32_t g = 0, sg = 0;  // group and stage within it of the stage being loaded
    for (uint32_t i = 0; i < nstep; ++i) {
      if (i < nstage) {
        DType *slot = ring[i % kDmaSlots];
#pragma unroll
        for (int q = 0; q < kDmaPerWave; ++q) {
          const uint32_t f0 = (q * kDmaLoaders + lw) * kWave * EPD;  // first element of this instruction
          const uint32_t seg = f0 / TL, off = f0 % TL;
          uint32_t n = g * SEGS + seg;
          uint32_t e = sg * TL + off + lane * EPD;
          n = n < n_out ? n : n_out - 1;  // clamped, never consumed
          e = e < seg_len ? e : seg_len - EPD;
          const uint32_t y = div_x.Div(e);
          const size_t row = static_cast<size_t>(n * n_keep + c) * n_y + y;
          LoadDwordToLds(src + row * stride + (e - y * n_x), slot + seg * LD + off);
        }
        if (++sg == stages_per_group) {
          sg = 0;
          ++g;
        }
        WaitStageLanded<Ring>();
      } else {
        WaitAllLanded();
      }
      BareBarrier();
    }
  } else {
    DType res, tres;
    Reducer::SetInitValue(res);
    Reducer::SetInitValue(tres);
    uint32_t g = 0, sg = 0;  // of the stage being folded
    for (uint32_t i = 0; i < nstep; ++i) {
      BareBarrier();
      if (i < static_cast<uint32_t>(kDmaAhead)) continue;
      const uint32_t st = i - kDmaAhead;
      const DType *slot = ring[st % kDmaSlots];
      const uint32_t e0 = sg * TL;
      const uint32_t live = (n_out - g * SEGS < (uint32_t)SEGS) ? n_out - g * SEGS : SEGS;
      if (lane < live) {
        const int count = (seg_len - e0 < (uint32_t)TL) ? static_cast<int>(seg_len - e0) : TL;
        ChainFold<Reducer>(tres, slot + lane * LD, 0, count);
      }
      if (++sg == stages_per_group) {
        /* the group's inner results are final: merge them in n order, then restart */
        for (uint32_t k = 0; k < live; ++k) {
          const DType v = WaveBroadcast(tres, static_cast<int>(k));
          Reducer::Reduce(res, v);
        }
        Reducer::SetInitValue(tres);
        sg = 0;
        ++g;
      }
    }
    if (lane == 0) Saver::template Save<DType>(dst[c], res * scale);
  }
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_REDUCE_DMA_H_
