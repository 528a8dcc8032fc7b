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

/* ------------------------------------------------------------------ KeepHighDim, split over n
 * The reference's order has two levels (mshadow/tensor_cpu-inl.h:230-268): an inner chain
 * per (n, c) segment, then a chain over n of the inner results. Only the second is tied to
 * the kept index c; the inner chains are independent of one another, so they are dealt out in
 * the order the segments lie in memory, SEGS neighbouring segments per workgroup (one chain
 * lane each), however few kept indices there are. The inner results go to a scratch array
 * `partial` of n_out * n_keep words; the workgroup that finishes last (counters in the
 * scratch memory, kSplitCounterWords words at `counter`, tell it so) folds them per kept index
 * in n order and saves the result; the counters are zero again when the launch ends. Launches that share a scratch array must not
 * overlap: the library hands one out per stream.
 *
 * A stage is one load instruction per segment: 64 lanes x 4 or 16 bytes of consecutive
 * elements, which land in LDS as they lie in memory, so a chain lane reads its operands four
 * at a time. 16-byte loads need rows of whole 16-byte packs (n_x, pitch, base); 4-byte loads
 * of 16-bit elements rows of whole pairs. */
template <int SEGS_, int LOADERS_, int SLOTS_, int WBYTES_>
struct SplitRing {
  static const int kSegs = SEGS_;
  static const int kLoaders = LOADERS_;
  static const int kSlots = SLOTS_;
  /*! \brief bytes a lane loads at a time: 4, or 16 where rows are whole 16-byte packs */
  static const int kLaneBytes = WBYTES_;
  static const int kAhead = SLOTS_ - 2;
  static const int kPerWave = SEGS_ / LOADERS_;
  static const int kThreads = (LOADERS_ + 1) * kWave;
  static_assert(SEGS_ % LOADERS_ == 0 && SEGS_ <= kWave, "one chain lane per segment");
  static_assert(kAhead >= 1 && kAhead * kPerWave < 64, "the wait-by-count immediate has 6 bits");
  static_assert(WBYTES_ == 4 || WBYTES_ == 16, "load width");
};
/*! \brief the configurations the library launches (measured on MI355X, sum over
 *  (64,64,112,112) / (256,16,112,112) floats: 54 / 71 us and 68 / 87 us, against 103 / 388 us
 *  with one workgroup per kept index): rows of whole 16-byte packs - 16 segments per
 *  workgroup, a kilobyte of each per stage; any rows - 32 segments, 256 bytes of each. */
typedef SplitRing<16, 8, 4, 16> HighDimSplitRingPacks;
/*! \brief ... and with more segments than 16 per CU: 32 per workgroup, one workgroup per CU
 *  (two workgroups of 16 on a CU ask for more than the CU's loads deliver: (128,64,112,112)
 *  took 105 us) */
typedef SplitRing<32, 8, 4, 16> HighDimSplitRingPacksWide;
typedef SplitRing<32, 8, 8, 4> HighDimSplitRing;

template <int BYTES>
__device__ __forceinline__ void LoadLaneToLds(const void *gsrc_of_lane, void *lds_wave_base) {
  const __attribute__((address_space(1))) void *from =
      (const __attribute__((address_space(1))) void *)gsrc_of_lane;
  __attribute__((address_space(3))) void *to = (__attribute__((address_space(3))) void *)lds_wave_base;
  if (BYTES == 16) {
    __builtin_amdgcn_global_load_lds(from, to, 16, 0, kDmaCachePolicy);
  } else {
    __builtin_amdgcn_global_load_lds(from, to, 4, 0, kDmaCachePolicy);
  }
}

/*! \brief the counters of the split reduction: a root and kSplitLeaves leaves, each in a cache
 *  line of its own (kSplitCounterStride words apart), all zero between launches */
const int kSplitLeaves = 64;
const int kSplitCounterStride = 32;
const int kSplitCounterWords = (1 + kSplitLeaves) * kSplitCounterStride;

/*! \brief words of scratch memory a launch needs for its inner results */
inline size_t SplitPartialWords(uint32_t n_out, uint32_t n_keep) {
  return static_cast<size_t>(n_out) * n_keep;
}

template <typename Saver, typename Reducer, typename DType, typename Ring>
__global__ void __launch_bounds__(Ring::kThreads)
    ReduceKeepHighDimSplitKernel(DType *dst, const DType *src, uint32_t stride, uint32_t n_out,
                                 uint32_t n_keep, uint32_t n_y, uint32_t n_x, FastDivU32 div_x,
                                 DType scale, uint32_t *partial, uint32_t *counter) {
  const int SEGS = Ring::kSegs, kSlots = Ring::kSlots, kAhead = Ring::kAhead, kPerWave = Ring::kPerWave;
  const int EPL = Ring::kLaneBytes / sizeof(DType);  // elements per lane and load
  const int TL = kWave * EPL;          // elements of a segment per stage
  const int LD = TL + 16 / sizeof(DType);  // chain lanes read words LD elements apart: no bank conflicts
  static_assert(sizeof(DType) == 4 || sizeof(DType) == 2, "a word of scratch memory holds a result");
  __shared__ MSHADOW_ALIGNED(16) DType ring[kSlots][SEGS * LD];
  __shared__ uint32_t i_am_last;

  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t nseg = n_out * n_keep;
  const uint32_t s0 = blockIdx.x * SEGS;
  const uint32_t live = (nseg - s0 < static_cast<uint32_t>(SEGS)) ? nseg - s0 : SEGS;
  const uint32_t seg_len = n_y * n_x;
  const uint32_t nstage = (seg_len + TL - 1) / TL;
  const uint32_t nstep = nstage == 0 ? 0 : nstage + kAhead;

  /* Which wave runs the chains: two workgroups share a CU where the ring is half the LDS, and
     two chain waves on one SIMD take turns (measured: 11.4 ns per add against 5.6 ns). The
     workgroups that meet on a CU differ in the lowest bit of their number or in bit 8. */
  const uint32_t chain_wave = (blockIdx.x ^ (blockIdx.x >> 8)) & 1u;
  if (wave != chain_wave) {
    const uint32_t lw = wave < chain_wave ? wave : wave - 1;
    for (uint32_t i = 0; i < nstep; ++i) {
      if (i < nstage) {
        DType *slot = ring[i % kSlots];
        uint32_t e = i * TL + lane * EPL;
        e = e < seg_len ? e : seg_len - EPL;  // clamped, never consumed
        const uint32_t y = div_x.Div(e);
        const size_t in_seg = static_cast<size_t>(y) * stride + (e - y * n_x);
#pragma unroll
        for (int q = 0; q < kPerWave; ++q) {
          const uint32_t seg = q * Ring::kLoaders + lw;
          const uint32_t sg = s0 + seg < nseg ? s0 + seg : nseg - 1;  // clamped likewise
          LoadLaneToLds<Ring::kLaneBytes>(src + static_cast<size_t>(sg) * n_y * stride + in_seg,
                                          slot + seg * LD);
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kAhead * kPerWave) : "memory");
      } else {
        WaitAllLanded();
      }
      BareBarrier();
    }
  } else {
    DType tres;
    Reducer::SetInitValue(tres);
    for (uint32_t i = 0; i < nstep; ++i) {
      BareBarrier();
      if (i < static_cast<uint32_t>(kAhead)) continue;
      const uint32_t st = i - kAhead;
      const uint32_t e0 = st * TL;
      if (lane < live) {
        const int count = (seg_len - e0 < (uint32_t)TL) ? static_cast<int>(seg_len - e0) : TL;
        ChainFold<Reducer>(tres, ring[st % kSlots] + lane * LD, 0, count);
      }
    }
    if (lane < live) {
      uint32_t bits = 0;
      __builtin_memcpy(&bits, static_cast<const void *>(&tres), sizeof(DType));
      __hip_atomic_store(partial + s0 + lane, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    /* The inner results must have reached the memory side before a counter moves. They are
       written through by device-scope stores, whose completion is what the wait below waits
       for; a release fence would do, but it also writes back this L2's every dirty line,
       once per workgroup. The last workgroup reads them with device-scope loads.
       Counting is in two levels, because increments of one address are served one after the
       other (about 40 ns each, which a thousand workgroups finishing together would wait
       for): workgroup b counts on leaf b % kSplitLeaves, and whoever completes a leaf counts
       on the root; whoever completes the root is last. A completed counter is cleared by the
       workgroup that completed it. */
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (lane == 0) {
      const uint32_t leaf = blockIdx.x % kSplitLeaves;
      const uint32_t in_leaf = (gridDim.x - leaf + kSplitLeaves - 1) / kSplitLeaves;
      const uint32_t leaves = gridDim.x < static_cast<uint32_t>(kSplitLeaves) ? gridDim.x : kSplitLeaves;
      uint32_t *leaf_counter = counter + (1 + leaf) * kSplitCounterStride;
      uint32_t last = 0u;
      if (__hip_atomic_fetch_add(leaf_counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
          in_leaf - 1u) {
        __hip_atomic_store(leaf_counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
            leaves - 1u) {
          last = 1u;
        }
      }
      i_am_last = last;
    }
  }
  __syncthreads();
  if (i_am_last == 0u) return;
  /* The merge: dst[c] = fold over n of the inner results, in n order. The results come in by
     device-scope loads, a tile of kMergeCols kept indices x as many n as the ring's memory
     holds at a time, all of a tile's loads in flight together (one after the other they would
     cost a trip to memory each); then thread c folds its column of the tile from LDS. */
  const int kMergeCols = 256;
  static_assert(Ring::kThreads >= kMergeCols, "a thread per kept index of a tile");
  uint32_t *tile = reinterpret_cast<uint32_t *>(&ring[0][0]);
  const uint32_t tile_words = sizeof(ring) / sizeof(uint32_t);
  const uint32_t tile_n = tile_words / kMergeCols;
  for (uint32_t c0 = 0; c0 < n_keep; c0 += kMergeCols) {
    const uint32_t c = c0 + threadIdx.x;
    DType res;
    Reducer::SetInitValue(res);
    for (uint32_t n0 = 0; n0 < n_out; n0 += tile_n) {
      const uint32_t nn = (n_out - n0 < tile_n) ? n_out - n0 : tile_n;
      for (uint32_t i = threadIdx.x; i < nn * kMergeCols; i += Ring::kThreads) {
        const uint32_t cc = c0 + i % kMergeCols;
        if (cc < n_keep) {
          tile[i] = __hip_atomic_load(partial + static_cast<size_t>(n0 + i / kMergeCols) * n_keep + cc,
                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      __syncthreads();
      if (threadIdx.x < static_cast<uint32_t>(kMergeCols) && c < n_keep) {
        for (uint32_t n = 0; n < nn; ++n) {
          const uint32_t bits = tile[n * kMergeCols + threadIdx.x];
          DType v;
          __builtin_memcpy(static_cast<void *>(&v), &bits, sizeof(DType));
          Reducer::Reduce(res, v);
        }
      }
      __syncthreads();
    }
    if (threadIdx.x < static_cast<uint32_t>(kMergeCols) && c < n_keep) {
      Saver::template Save<DType>(dst[c], res * scale);
    }
  }
  if (threadIdx.x == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_REDUCE_DMA_H_
