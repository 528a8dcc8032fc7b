/*
 * Reduce-to-1D kernels that keep the CPU path's order of operations.
 *
 * The reference CPU path (mshadow/tensor_cpu-inl.h:203-268) gives every output to one
 * thread that folds its inputs strictly in order:
 *   KeepLowest   dst[x] = scale * (((src(0,x) + src(1,x)) + src(2,x)) + ...)
 *   KeepHighDim  dst[c] = scale * fold_n( fold_{y,x} src(n,c,y,x) )   (two levels)
 * A float sum depends on that order, and the difference to a tree sum exceeds 1e-5
 * relative on outputs near zero, so these kernels keep it: each output (or each inner
 * (n, c) segment) is a serial chain of dependent adds owned by ONE lane. Bandwidth
 * comes from everything around the chain:
 *   - all threads of a workgroup (1024 for long reductions) stream the next tiles from
 *     HBM with coalesced loads (16 independent loads per thread in flight, two stages
 *     deep: up to 128 KB per CU), and drop them into LDS transposed, so that
 *   - the chain lanes of wave 0 read their own next 4 operands with one ds_read_b128
 *     and spend one dependent add per element.
 * Work is split so that every CU owns a few chains (16 columns, or one kept index, per
 * workgroup) instead of one CU owning many. The reference's GPU kernels
 * (MapRedKeepLowestKernel / MapReduceKeepDim1Kernel, cuda/tensor_gpu-inl.cuh:122-215)
 * tree-reduce in shared memory with a 32-lane tail; they are replaced, not ported.
 *
 * Algorithmic traffic: sizeof(DType) bytes per input element, read once; HBM-bound.
 * The chain costs about one VALU issue slot per input row (KeepLowest) which at
 * 16384 rows is of the same order as the HBM time, see the design notes.
 */
#ifndef MSHADOW_HIP_KERNELS_REDUCE_H_
#define MSHADOW_HIP_KERNELS_REDUCE_H_

#include "../../core/fastdiv.h"
#include "../../expr/plan.h"
#include "./common.h"

namespace mshadow {
namespace hip {

/*! \brief loads per thread per stage (all issued before any is consumed) */
const int kRedDepth = 16;
/*! \brief columns per workgroup in KeepLowest: 16 floats = one 64-byte segment per row */
const int kLowestCols = 16;
/*! \brief workgroup sizes: the large one keeps 64 KB of loads in flight per stage and is
 *  used when the reduction is long enough to fill its pipeline */
const int kRedBlockSmall = 256;
const int kRedBlockLarge = 1024;
/*! \brief the large workgroup for element type DType: its two staging tiles hold
 *  2 * THREADS * kRedDepth elements, which for 8-byte types fits the 160 KB of LDS only with
 *  the small workgroup */
template <typename DType>
struct RedBlockLargeFor {
  static const int value = sizeof(DType) <= 4 ? kRedBlockLarge : kRedBlockSmall;
};

/*! \brief value of v in lane `lane` for any small trivially copyable type */
template <typename DType>
__device__ __forceinline__ DType WaveBroadcast(DType v, int lane) {
  const int kWords = (sizeof(DType) + 3) / 4;
  uint32_t w[kWords];
#pragma unroll
  for (int i = 0; i < kWords; ++i) w[i] = 0;
  __builtin_memcpy(w, &v, sizeof(DType));
#pragma unroll
  for (int i = 0; i < kWords; ++i) w[i] = ReadLaneU32(w[i], lane);
  DType r;
  __builtin_memcpy(&r, w, sizeof(DType));
  return r;
}

/*! \brief fold this lane's elements [begin, count) into res, in order. Element r lives at
 *  vals[(r / 4) * GSTRIDE + r % 4]: groups of four consecutive elements are contiguous
 *  (one 128-bit LDS read), GSTRIDE floats apart (4 = fully contiguous). The operands of
 *  the next 32 steps are fetched from LDS (eight 128-bit reads) while the current 32
 *  dependent reductions execute, so a step costs one VALU issue plus a quarter of an LDS
 *  read. */
template <typename Reducer, typename DType, int PACKS, int GSTRIDE>
__device__ __forceinline__ void ChainLoad(expr::Pack<DType, 4> (&dst)[PACKS], const DType *src) {
#pragma unroll
  for (int i = 0; i < PACKS; ++i) {
    dst[i] = *reinterpret_cast<const expr::Pack<DType, 4> *>(src + GSTRIDE * i);
  }
}
template <typename Reducer, typename DType, int PACKS>
__device__ __forceinline__ void ChainApply(DType &res, const expr::Pack<DType, 4> (&p)[PACKS]) {
#pragma unroll
  for (int i = 0; i < PACKS; ++i) {
    Reducer::Reduce(res, p[i].v[0]);
    Reducer::Reduce(res, p[i].v[1]);
    Reducer::Reduce(res, p[i].v[2]);
    Reducer::Reduce(res, p[i].v[3]);
  }
}

template <typename Reducer, int GSTRIDE = 4, typename DType>
__device__ __forceinline__ void ChainFold(DType &res, const DType *vals, int begin, int count) {
  typedef expr::Pack<DType, 4> P4;
  const int kBlk = 32;
  const int kPacks = kBlk / 4;
  const int kBlkStride = kPacks * GSTRIDE;  // floats between consecutive blocks of 32
#define MSHADOW_CHAIN_AT(r) vals[((r) >> 2) * GSTRIDE + ((r) & 3)]
  int r = begin;
  for (; r < count && (r & (kBlk - 1)); ++r) Reducer::Reduce(res, MSHADOW_CHAIN_AT(r));
  if (r + kBlk <= count) {
    /* two register sets alternate: while one is being folded the other is in flight */
    const DType *blk = vals + (r >> 2) * GSTRIDE;
    P4 a[kPacks], b[kPacks];
    ChainLoad<Reducer, DType, kPacks, GSTRIDE>(a, blk);
    for (; r + 3 * kBlk <= count; r += 2 * kBlk, blk += 2 * kBlkStride) {
      ChainLoad<Reducer, DType, kPacks, GSTRIDE>(b, blk + kBlkStride);
      __builtin_amdgcn_sched_barrier(0);
      ChainApply<Reducer, DType, kPacks>(res, a);
      ChainLoad<Reducer, DType, kPacks, GSTRIDE>(a, blk + 2 * kBlkStride);
      __builtin_amdgcn_sched_barrier(0);
      ChainApply<Reducer, DType, kPacks>(res, b);
    }
    if (r + 2 * kBlk <= count) {
      ChainLoad<Reducer, DType, kPacks, GSTRIDE>(b, blk + kBlkStride);
      __builtin_amdgcn_sched_barrier(0);
      ChainApply<Reducer, DType, kPacks>(res, a);
      ChainApply<Reducer, DType, kPacks>(res, b);
      r += 2 * kBlk;
    } else {
      ChainApply<Reducer, DType, kPacks>(res, a);
      r += kBlk;
    }
  }
  for (; r < count; ++r) Reducer::Reduce(res, MSHADOW_CHAIN_AT(r));
#undef MSHADOW_CHAIN_AT
}

/* ------------------------------------------------------------------ KeepLowest */
template <typename Saver, typename Reducer, typename DType, int THREADS, typename DPlan,
          typename SPlan>
__global__ void __launch_bounds__(THREADS)
    ReduceKeepLowestKernel(DPlan dplan, SPlan splan, uint32_t rows, uint32_t cols, DType scale) {
  const int CW = kLowestCols;
  const int RPP = THREADS / CW;      // rows covered by one load pass of the workgroup
  const int TR = RPP * kRedDepth;    // rows per stage
  const int LD = TR + 4;             // pitch of one column in the transposed tile
  __shared__ MSHADOW_ALIGNED(16) DType tile[2][CW * LD];

  const int t = threadIdx.x;
  const int col = t % CW;
  const int rsub = t / CW;
  const uint32_t x = StripOfBlock(blockIdx.x, gridDim.x) * CW + col;
  const bool col_ok = x < cols;
  const uint32_t nstage = (rows + TR - 1) / TR;
  const bool chain_lane = (t < CW) && col_ok;  // lanes 0..CW-1 of wave 0 own the chains

  /* loads are never predicated: out-of-range rows / columns re-read the last valid one
     (their values are not consumed), so every stage issues exactly kRedDepth loads and
     the wait before the LDS write can leave the next stage's loads in flight */
  const uint32_t xc = col_ok ? x : cols - 1;
  const uint32_t last_row = rows - 1;
  DType cur[kRedDepth], nxt[kRedDepth];
#pragma unroll
  for (int k = 0; k < kRedDepth; ++k) {
    const uint32_t r = rsub + RPP * k;
    nxt[k] = splan.Eval(r < rows ? r : last_row, xc);
  }
  DType res = DType(0);
  for (uint32_t st = 0; st < nstage; ++st) {
    const uint32_t row0 = st * TR;
    /* take delivery of this stage's loads, then put the next stage's in flight; they
       travel while wave 0 runs the chain below */
#pragma unroll
    for (int k = 0; k < kRedDepth; ++k) cur[k] = nxt[k];
    if (st + 1 < nstage) {
#pragma unroll
      for (int k = 0; k < kRedDepth; ++k) {
        const uint32_t r = row0 + TR + rsub + RPP * k;
        nxt[k] = splan.Eval(r < rows ? r : last_row, xc);
      }
    }
    DType *buf = tile[st & 1];
#pragma unroll
    for (int k = 0; k < kRedDepth; ++k) buf[col * LD + rsub + RPP * k] = cur[k];
    __syncthreads();
    if (chain_lane) {
      const DType *mine = buf + t * LD;
      const int count = (rows - row0 < (uint32_t)TR) ? static_cast<int>(rows - row0) : TR;
      int begin = 0;
      if (st == 0) {  // the reference starts from src(0, x), not from an initial value
        res = mine[0];
        begin = 1;
      }
      ChainFold<Reducer>(res, mine, begin, count);
    }
  }
  if (chain_lane) Saver::template Save<DType>(dplan.REval(0, x), res * scale);
}

/* ------------------------------------------------------------------ KeepHighDim */
/* shape viewed as (n_out, n_keep, n_y, n_x); one workgroup per kept index c. SEGS inner
   segments (n values) are staged side by side, one chain lane each. */
template <typename Saver, typename Reducer, typename DType, int THREADS, int SEGS, typename DPlan,
          typename SPlan>
__global__ void __launch_bounds__(THREADS)
    ReduceKeepHighDimKernel(DPlan dplan, SPlan splan, uint32_t n_out, uint32_t n_keep,
                            uint32_t n_y, uint32_t n_x, FastDivU32 div_x, DType scale) {
  const int TL = THREADS * kRedDepth / SEGS;  // elements of each segment per stage
  const int LD = TL + 4;
  __shared__ MSHADOW_ALIGNED(16) DType tile[2][SEGS * LD];

  const int t = threadIdx.x;
  const uint32_t c = blockIdx.x;
  const uint32_t seg_len = n_y * n_x;
  const uint32_t stages_per_group = (seg_len + TL - 1) / TL;
  const uint32_t groups = (n_out + SEGS - 1) / SEGS;
  const uint32_t nstage = groups * stages_per_group;
  const bool chain_lane = t < SEGS;

  DType cur[kRedDepth], nxt[kRedDepth];
#define MSHADOW_HIGHDIM_LOAD(REGS, STAGE)                                              \
  {                                                                                    \
    const uint32_t g_ = (STAGE) / stages_per_group;                                    \
    const uint32_t e0_ = ((STAGE) - g_ * stages_per_group) * TL;                       \
    _Pragma("unroll") for (int k = 0; k < kRedDepth; ++k) {                            \
      const uint32_t f_ = k * THREADS + t;                                             \
      uint32_t n_ = g_ * SEGS + f_ / TL;                                               \
      uint32_t e_ = e0_ + f_ % TL;                                                     \
      /* never predicated (see KeepLowest): clamp to the last valid element */         \
      n_ = n_ < n_out ? n_ : n_out - 1;                                                \
      e_ = e_ < seg_len ? e_ : seg_len - 1;                                            \
      const uint32_t y_ = div_x.Div(e_);                                               \
      REGS[k] = splan.Eval((n_ * n_keep + c) * n_y + y_, e_ - y_ * n_x);               \
    }                                                                                  \
  }
  if (nstage > 0) MSHADOW_HIGHDIM_LOAD(nxt, 0u)
  DType res, tres;
  Reducer::SetInitValue(res);
  Reducer::SetInitValue(tres);
  for (uint32_t st = 0; st < nstage; ++st) {
#pragma unroll
    for (int k = 0; k < kRedDepth; ++k) cur[k] = nxt[k];
    if (st + 1 < nstage) MSHADOW_HIGHDIM_LOAD(nxt, st + 1)
    DType *buf = tile[st & 1];
#pragma unroll
    for (int k = 0; k < kRedDepth; ++k) {
      const uint32_t f = k * THREADS + t;
      buf[(f / TL) * LD + f % TL] = cur[k];
    }
    __syncthreads();
    if (t < kWave) {  // wave 0: lanes < SEGS chain, all 64 take part in the broadcast below
      const uint32_t g = st / stages_per_group;
      const uint32_t sg = st - g * stages_per_group;
      const uint32_t e0 = sg * TL;
      const uint32_t live = (n_out - g * SEGS < (uint32_t)SEGS) ? n_out - g * SEGS : SEGS;
      if (chain_lane && static_cast<uint32_t>(t) < live) {
        const int count = (seg_len - e0 < (uint32_t)TL) ? static_cast<int>(seg_len - e0) : TL;
        ChainFold<Reducer>(tres, buf + t * LD, 0, count);
      }
      if (sg + 1 == stages_per_group) {
        /* the group's inner results are final: merge them in n order, then restart */
        for (uint32_t i = 0; i < live; ++i) {
          const DType v = WaveBroadcast(tres, static_cast<int>(i));
          Reducer::Reduce(res, v);
        }
        Reducer::SetInitValue(tres);
      }
    }
  }
#undef MSHADOW_HIGHDIM_LOAD
  if (t == 0) Saver::template Save<DType>(dplan.REval(0, c), DType(res * scale));
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_REDUCE_H_
