/*
 * Row softmax and its gradient for gfx950.
 *
 * SoftmaxRowKernel: one workgroup per row, the whole row held in registers, so HBM
 * sees one read of src and one write of dst (2 * 4 bytes per element; the reference
 * kernel, mshadow/cuda/tensor_gpu-inl.cuh:330-393, moves 5). Steps per row:
 *   1. 128-bit loads, row maximum by DPP wave reduction + one LDS exchange;
 *   2. p = exp(x - max) in registers (hardware exp2 with a compensated argument);
 *   3. the row sum in the CPU path's left-to-right order (ordered_sum.h: planned from
 *      approximate prefix sums, exact integer adds inside a binade, a short ordered
 *      walk over the chunks where a power of two is crossed), so that the sum is, bit
 *      for bit, what mshadow/tensor_cpu-inl.h:277-281 computes from the same p;
 *   4. p / sum (reciprocal and one correction step), 128-bit stores.
 * dst may alias src (every element is read before the row is written).
 * SoftmaxLongRowKernel covers rows too long for registers with the same arithmetic,
 * staging p through dst. SoftmaxGradKernel is a 128-bit copy with one element per row
 * decremented (mshadow/tensor_cpu-inl.h:287-302).
 */
#ifndef MSHADOW_AMD_CSRC_SOFTMAX_KERNELS_H_
#define MSHADOW_AMD_CSRC_SOFTMAX_KERNELS_H_

#include <hip/hip_runtime.h>

#include <mshadow/core/fastdiv.h>
#include <mshadow/hip/kernels/common.h>

#include "ordered_sum.h"
#include "stream_access.h"

namespace mshadow_hipk {

using mshadow::hip::kWave;
using mshadow::hip::LaneId;
using mshadow::hip::ReadLaneF32;
using mshadow::hip::WaveId;
using mshadow::hip::WaveInclusiveScanF32;
using mshadow::hip::WaveMaxF32;

/*! \brief LDS scratch of the ordered sum: two alternating sets of per-wave totals and
 *  the hand-over slot for the running sum */
template <int WAVES>
struct OrderedSumLds {
  float q[2][WAVES];
  float s;
  float wmax[WAVES];
};

/*! \brief one wave adds its 64 * N terms (lane order, then element order) to s exactly
 *  as a serial loop would; called only for the wave in which a chunk was rejected */
template <int N>
__device__ inline float WaveResolve(float s, const float (&t)[N]) {
  using namespace ordered_sum;
  const int lane = LaneId();
  int start = 0;
  while (true) {
    const Binade b = BinadeOf(s);
    const float q = (lane >= start) ? LaneQuant<N>(t, b) : 0.0f;
    const float incl = WaveInclusiveScanF32(q);
    const bool fail = (lane >= start) && !Fits(b, incl);
    const unsigned long long mask = __ballot(fail);
    if (mask == 0ull) return Accept(s, b, ReadLaneF32(incl, kWave - 1));
    const int first = __ffsll(mask) - 1;
    /* lanes before `first` are exact integer adds (their inclusive prefix is exact) */
    s = Accept(s, b, first > 0 ? ReadLaneF32(incl, first - 1) : 0.0f);
    /* lane `first` does real float adds; every lane computes, one result is taken */
    s = ReadLaneF32(TrueAdd<N>(s, t), first);
    start = first + 1;
    if (start == kWave) return s;
  }
}

/*! \brief block-wide: add one slab (THREADS * N consecutive terms, thread-major) to s.
 *  s is uniform over the block on entry and on exit. `buf` alternates the LDS slot. */
template <int THREADS, int N>
__device__ inline float BlockOrderedAdd(float s, const float (&t)[N],
                                        OrderedSumLds<THREADS / kWave> *lds, int *buf) {
  using namespace ordered_sum;
  const int W = THREADS / kWave;
  const int wave = WaveId();
  const int lane = LaneId();
  int pos = 0;  // waves before pos are already in s
  while (true) {
    const Binade b = BinadeOf(s);
    if (wave >= pos) {
      const float q = ReadLaneF32(WaveInclusiveScanF32(LaneQuant<N>(t, b)), kWave - 1);
      if (lane == 0) lds->q[*buf][wave] = q;
    }
    __syncthreads();
    /* the per-wave totals are scanned across lanes (lane w holds wave w's total): the
       first wave whose inclusive prefix leaves the binade is the one to resolve */
    const float qv = (lane < W && lane >= pos) ? lds->q[*buf][lane] : 0.0f;
    const float incl = WaveInclusiveScanF32(qv);
    const bool over = lane < W && lane >= pos && !Fits(b, incl);
    const unsigned long long mask = __ballot(over);
    const int failw = mask ? __ffsll(mask) - 1 : W;
    const float acc = failw > 0 ? ReadLaneF32(incl, failw - 1) : 0.0f;
    *buf ^= 1;
    s = Accept(s, b, acc);
    if (failw == W) return s;
    if (wave == failw) {
      const float r = WaveResolve<N>(s, t);
      if (lane == 0) lds->s = r;
    }
    __syncthreads();
    s = lds->s;
    pos = failw + 1;
    if (pos == W) return s;
  }
}

/* ---- planned row sum (registers hold the whole row) ---------------------------------
 * Thread layout: wave w owns a contiguous W-th of the row, slab j of it is the chunk
 * k = w * SLABS + j (64 * N consecutive terms, lane-major). See ordered_sum.h for the
 * plan; the steps here are
 *   A  every wave: approximate sum of each of its chunks -> LDS            (barrier)
 *   B  every wave (redundantly): prefix over all chunks, plan per chunk
 *   C  every wave: quantise its clean chunks, integer totals -> LDS; its dirty chunks
 *      are parked, with their terms, in LDS slots                          (barrier)
 *   D  every wave: integer prefix over the clean chunks; all waves together: a plan per
 *      lane for each parked chunk, and the order of the slots in the row   (barrier)
 *      wave 0: for each parked chunk in row order, apply the clean run in front of it
 *      and walk it (runs of clean lanes as integers, the other lanes term by term),
 *      fetching the next slot meanwhile                                    (barrier)
 *   E  every wave: apply the clean run behind the last dirty chunk.
 * A row with more dirty chunks than slots is summed by wave scans instead (as is a row
 * whose plan fails a verification).
 * Lane l keeps the chunk-table entries of chunks l * CPL .. l * CPL + CPL - 1. */
const uint32_t kDirtyQ = 0xffffffffu;
/*! \brief lanes of a row's first chunk that are added serially without a plan */
const int kHeadLanes = 32;
/*! \brief dirty chunks per row with a lane-level plan parked in LDS (a row of softmax
 *  terms has about a dozen); further ones are resolved by wave scans */
const int kPlanSlots = 24;

/* hook for a profiling build: a translation unit may define this to record a timestamp
   at the boundaries of the steps; it is empty in the library */
#ifndef MSHADOW_ROWSUM_STAMP
#define MSHADOW_ROWSUM_STAMP(step)
#endif

/*! \brief lane-level plan of one dirty chunk, parked in LDS between steps C and D, with
 *  the chunk's terms (so that the walk needs nothing from the register-resident row).
 *  General chunk: a = integer total of the clean lanes in front of the lane, b = its plan
 *  code. Two-binade chunk: a / b = inclusive integer prefix of the lanes quantised against
 *  the lower / upper binade (lanes holding a tie count as 0). */
template <int N>
struct LanePlanSlot {
  float t[kWave][N];
  uint32_t a[kWave];
  uint32_t b[kWave];
  unsigned long long tie_lo, tie_hi;  //!< two-binade chunks: lanes holding a tie (lower / upper binade)
  uint32_t total;  //!< general chunks: integer total of the clean lanes
  int kind;        //!< plan code of the chunk (kPlanWalk or kPlanTwoBinades + e)
  float start;     //!< approximate prefix sum in front of the chunk
  int chunk;       //!< index of the chunk in the row
  uint32_t ex;     //!< integer total of the clean chunks in front of this one
  int e_run;       //!< binade of the clean chunk just in front (if there is one)
};

template <int W, int SLABS, int N>
struct RowSumLds {
  /* small workgroups share a CU with several others: fewer slots each */
  static const int kWanted = W <= 4 ? kPlanSlots * 2 / 3 : kPlanSlots;
  static const int kSlots = (W * SLABS < kWanted) ? W * SLABS : kWanted;
  float approx[W * SLABS];
  uint32_t q[W * SLABS];
  float s;       //!< running sum handed from wave to wave
  uint32_t ex;   //!< integer prefix (over clean chunks) already applied to s
  int fail;      //!< a verification failed: redo the row the slow way
  uint32_t nslots;  //!< plan slots handed out
  float wmax[W];
  /*! \brief the plan slots in the order of their chunks in the row */
  signed char order[kSlots];
  LanePlanSlot<N> plan[kSlots];
};

/*! \brief plan code of a piece that stays in one binade */
__device__ __forceinline__ bool IsClean(int code) {
  return code >= 0 && code < ordered_sum::kPlanTwoBinades;
}

/*! \brief entry k of a table spread over lanes (CPL entries per lane); k is uniform */
template <int CPL>
__device__ __forceinline__ uint32_t TableAt(const uint32_t (&a)[CPL], int k) {
  /* every slot is read from the lane first and the choice made among the scalars: a
     choice among the per-lane registers would be turned into an indexed private array */
  uint32_t v = mshadow::hip::ReadLaneU32(a[0], k / CPL);
#pragma unroll
  for (int c = 1; c < CPL; ++c) {
    const uint32_t o = mshadow::hip::ReadLaneU32(a[c], k / CPL);
    v = (k % CPL == c) ? o : v;
  }
  return v;
}

/*! \brief slab j of the register-resident row (j uniform, not a compile-time constant):
 *  a binary tree of uniform branches, log2(SLABS) deep */
template <int LO, int HI, int SLABS, int N>
struct SlabPicker {
  static __device__ __forceinline__ void Pick(float (&t)[N], const float (&v)[SLABS][N], int j) {
    const int MID = (LO + HI) / 2;
    if (j < MID) {
      SlabPicker<LO, MID, SLABS, N>::Pick(t, v, j);
    } else {
      SlabPicker<MID, HI, SLABS, N>::Pick(t, v, j);
    }
  }
};
template <int LO, int SLABS, int N>
struct SlabPicker<LO, LO + 1, SLABS, N> {
  static __device__ __forceinline__ void Pick(float (&t)[N], const float (&v)[SLABS][N], int) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      t[i] = v[LO][i];
      /* keeps the tree a tree: folded into one indexed access, the whole row would move
         from registers to scratch memory */
      asm volatile("" : "+v"(t[i]));
    }
  }
};
template <int SLABS, int N>
__device__ __forceinline__ void SelectSlab(float (&t)[N], const float (&v)[SLABS][N], int j) {
  SlabPicker<0, SLABS, SLABS, N>::Pick(t, v, j);
}

/*! \brief lane-level plan of one chunk whose approximate prefix sum in front is `start`:
 *  *code = binade the lane's terms stay in, or kPlanWalk; *ex = integer total of the
 *  clean lanes in front of this lane; returns the integer total of all clean lanes */
template <int N>
__device__ __forceinline__ uint32_t PlanLanes(const float (&t)[N], float start, float margin,
                                              bool head, uint32_t *ex, int *code) {
  using namespace ordered_sum;
  float a = t[0];
#pragma unroll
  for (int i = 1; i < N; ++i) a += t[i];
  const float incl = WaveInclusiveScanF32(a);
  int c = PlanLane(start + (incl - a), start + incl, margin);
  /* the head of a row (the sum starts at zero): its first lanes cross a binade or hold a
     tie nearly every time and are added term by term without asking */
  if (head && LaneId() < kHeadLanes) c = kPlanWalk;
  float q = 0.0f;
  if (c >= 0) {
    q = LaneQuant<N>(t, BinadeOfExponent(static_cast<uint32_t>(c)));
    if (!(q < kLimit)) c = kPlanWalk;  // a tie (or a term the plan did not expect)
  }
  /* neighbouring clean lanes must agree on the binade, or the later one is walked */
  const int before = __shfl_up(c, 1);
  if (LaneId() > 0 && c >= 0 && before >= 0 && before != c) c = kPlanWalk;
  const uint32_t qi = c >= 0 ? static_cast<uint32_t>(q) : 0u;
  const uint32_t inclu = mshadow::hip::WaveInclusiveScanU32(qi);
  *ex = inclu - qi;
  *code = c;
  return mshadow::hip::ReadLaneU32(inclu, kWave - 1);
}

/*! \brief s plus the terms of lanes 0 .. kHeadLanes-1 of a chunk parked in LDS (t[lane][i]),
 *  one float add after the other. Every lane reads the same addresses (an LDS broadcast),
 *  so the operands arrive in vector registers and the only chain is the adds themselves. */
template <int N>
__device__ __forceinline__ float HeadSerialAdd(float s, const float (*t)[N]) {
  const int kBatch = 4;  // lanes whose terms are fetched before they are added
#pragma unroll
  for (int l0 = 0; l0 < kHeadLanes; l0 += kBatch) {
    float r[kBatch][N];
#pragma unroll
    for (int l = 0; l < kBatch; ++l) {
#pragma unroll
      for (int i = 0; i < N; ++i) r[l][i] = t[l0 + l][i];
    }
#pragma unroll
    for (int l = 0; l < kBatch; ++l) {
#pragma unroll
      for (int i = 0; i < N; ++i) s = s + r[l][i];
    }
  }
  return s;
}

/*! \brief s plus one chunk, given its lane-level plan: runs of clean lanes are applied as
 *  integers (and verified), runs of other lanes add their terms one by one. `skip` names
 *  lanes that are in s already. */
template <int N>
__device__ __forceinline__ float WalkLanes(float s, const float (&t)[N], uint32_t ex, int code,
                                           uint32_t total, unsigned long long skip, bool *fail) {
  using namespace ordered_sum;
  using mshadow::hip::ReadLaneU32;
  unsigned long long todo = __ballot(code < 0) & ~skip;
  uint32_t done = 0u;
  while (todo != 0ull) {
    const int l0 = __ffsll(static_cast<long long>(todo)) - 1;
    const uint32_t exl = ReadLaneU32(ex, l0);
    if (exl != done) {
      s = FlushRun(s, static_cast<int>(ReadLaneU32(static_cast<uint32_t>(code), l0 - 1)), exl - done, fail);
      done = exl;
    }
    /* the lanes l0 .. l1-1 are walked: l1 = first clean lane above l0 (or 64) */
    const unsigned long long above = ~(todo >> l0);
    const int len = above != 0ull ? __ffsll(static_cast<long long>(above)) - 1 : kWave - l0;
    const int l1 = l0 + len;
    for (int l = l0; l < l1; ++l) {
#pragma unroll
      for (int i = 0; i < N; ++i) s = s + ReadLaneF32(t[i], l);
    }
    todo = l1 < kWave ? (todo >> l1) << l1 : 0ull;
  }
  if (total != done) {
    s = FlushRun(s, static_cast<int>(ReadLaneU32(static_cast<uint32_t>(code), kWave - 1)), total - done, fail);
  }
  return s;
}

/*! \brief plan of a chunk that starts in binade elo and may end in elo + 1: every lane
 *  quantised against both; a lane holding a tie under a binade counts as 0 in that prefix
 *  and is named in the tie mask */
template <int N>
__device__ __forceinline__ void PlanTwoBinades(const float (&t)[N], int elo, uint32_t *incl_lo,
                                               uint32_t *incl_hi, unsigned long long *tie_lo,
                                               unsigned long long *tie_hi) {
  using namespace ordered_sum;
  const float qlo = LaneQuant<N>(t, BinadeOfExponent(static_cast<uint32_t>(elo)));
  const float qhi = LaneQuant<N>(t, BinadeOfExponent(static_cast<uint32_t>(elo + 1)));
  const bool tlo = !(qlo < kLimit), thi = !(qhi < kLimit);
  *incl_lo = mshadow::hip::WaveInclusiveScanU32(tlo ? 0u : static_cast<uint32_t>(qlo));
  *incl_hi = mshadow::hip::WaveInclusiveScanU32(thi ? 0u : static_cast<uint32_t>(qhi));
  *tie_lo = __ballot(tlo);
  *tie_hi = __ballot(thi);
}

/*! \brief s plus one chunk planned by PlanTwoBinades. Each round accepts, as integers,
 *  the lanes up to the first one that holds a tie or would carry the sum out of the
 *  current binade, adds that lane's terms one by one, and goes on - against the upper
 *  binade once the sum has crossed. A crossing chunk takes two rounds. */
template <int N>
__device__ __forceinline__ float WalkTwoBinades(float s, const float (&t)[N], int elo,
                                                uint32_t incl_lo, uint32_t incl_hi,
                                                unsigned long long tie_lo,
                                                unsigned long long tie_hi, bool *fail) {
  using namespace ordered_sum;
  using mshadow::hip::ReadLaneU32;
  /* The usual course in straight-line code: the lanes up to the crossing (or tie) lane f
     as integers in the lower binade, lane f term by term, all lanes behind it as integers
     in whichever of the two binades the sum is in then. Anything else (a second tie, a sum
     in neither binade) takes the general rounds below from the start. */
  {
    const uint32_t el = static_cast<uint32_t>(elo);
    const float m = s * FloatOf((277u - el) << 23);
    const uint32_t room = 16777216u - static_cast<uint32_t>(m);
    const unsigned long long ev = __ballot(incl_lo >= room) | tie_lo;
    const bool in_lo = m >= 8388608.0f && m < kLimit;
    if (in_lo && ev == 0ull) {
      return (m + static_cast<float>(ReadLaneU32(incl_lo, kWave - 1))) * FloatOf((el - 23u) << 23);
    }
    if (in_lo) {
      const int f = __ffsll(static_cast<long long>(ev)) - 1;
      const uint32_t upto = f > 0 ? ReadLaneU32(incl_lo, f - 1) : 0u;
      float s2 = (m + static_cast<float>(upto)) * FloatOf((el - 23u) << 23);
#pragma unroll
      for (int i = 0; i < N; ++i) s2 = s2 + ReadLaneF32(t[i], f);
      const float mh = s2 * FloatOf((276u - el) << 23);  // in units of the upper binade
      const bool up = mh >= 8388608.0f;
      const float m2 = up ? mh : mh + mh;                 // exact either way
      const uint32_t incl2 = up ? incl_hi : incl_lo;
      const uint32_t base2 = ReadLaneU32(incl2, f);
      const uint32_t room2 = 16777216u - static_cast<uint32_t>(m2);
      const unsigned long long behind = f < kWave - 1 ? (~0ull << 1) << f : 0ull;
      const unsigned long long ev2 = (__ballot(incl2 - base2 >= room2) | (up ? tie_hi : tie_lo)) & behind;
      if (ev2 == 0ull && m2 >= 8388608.0f && m2 < kLimit) {
        const float u2 = FloatOf((el - 23u + (up ? 1u : 0u)) << 23);
        return (m2 + static_cast<float>(ReadLaneU32(incl2, kWave - 1) - base2)) * u2;
      }
    }
  }
  unsigned long long pending = ~0ull;  // lanes not yet in s
  int p = 0;                           // = number of lanes in s
  bool hi = false;                     // s has crossed into the upper binade
  while (true) {
    const uint32_t e = static_cast<uint32_t>(elo) + (hi ? 1u : 0u);
    const float m = s * FloatOf((277u - e) << 23);
    if (!hi && !(m < kLimit)) {
      hi = true;
      continue;
    }
    if (!(m >= 8388608.0f && m < kLimit)) {  // s is in neither binade: the plan was wrong
      *fail = true;
      return s;
    }
    const float u = FloatOf((e - 23u) << 23);
    const uint32_t incl = hi ? incl_hi : incl_lo;
    const uint32_t base = p > 0 ? ReadLaneU32(incl, p - 1) : 0u;
    const uint32_t room = 16777216u - static_cast<uint32_t>(m);  // integer steps left in the binade
    /* lanes already in s compare on a wrapped difference; `pending` masks them out */
    const unsigned long long events = (__ballot(incl - base >= room) | (hi ? tie_hi : tie_lo)) & pending;
    if (events == 0ull) return (m + static_cast<float>(ReadLaneU32(incl, kWave - 1) - base)) * u;
    const int f = __ffsll(static_cast<long long>(events)) - 1;
    const uint32_t upto = f > 0 ? ReadLaneU32(incl, f - 1) : 0u;
    s = (m + static_cast<float>(upto - base)) * u;
#pragma unroll
    for (int i = 0; i < N; ++i) s = s + ReadLaneF32(t[i], f);
    if (f == kWave - 1) return s;
    p = f + 1;
    pending = (~0ull << 1) << f;
  }
}

template <int THREADS, int SLABS, int N>
__device__ inline float RowOrderedSum(const float (&v)[SLABS][N], int cols,
                                      RowSumLds<THREADS / kWave, SLABS, N> *lds) {
  using namespace ordered_sum;
  using mshadow::hip::ReadLaneU32;
  using mshadow::hip::WaveInclusiveScanU32;
  typedef RowSumLds<THREADS / kWave, SLABS, N> Lds;
  const int W = THREADS / kWave;
  const int NCH = W * SLABS;
  const int CPL = (NCH + kWave - 1) / kWave;
  static_assert(NCH % CPL == 0 && SLABS % CPL == 0, "chunk table does not tile the lanes");
  static_assert(SLABS <= 32, "the per-wave dirty mask has 32 bits");
  const int wave = __builtin_amdgcn_readfirstlane(WaveId());
  const int lane = LaneId();
  const float margin = PlanMargin(cols);

  /* A: approximate chunk sums */
  MSHADOW_ROWSUM_STAMP(0)
  if (threadIdx.x == 0) {
    lds->s = 0.0f;
    lds->ex = 0u;
    lds->fail = 0;
    lds->nslots = 0u;
  }
  {
    float part[SLABS];
#pragma unroll
    for (int j = 0; j < SLABS; ++j) {
      part[j] = v[j][0];
#pragma unroll
      for (int i = 1; i < N; ++i) part[j] += v[j][i];
    }
    const float mine = mshadow::hip::WaveSumMany<SLABS>(part);  // lane l: chunk l % SLABS
    if (lane < SLABS) lds->approx[wave * SLABS + lane] = mine;
  }
  __syncthreads();
  MSHADOW_ROWSUM_STAMP(1)

  /* B: plan per chunk, identical in every wave */
  uint32_t code[CPL];   // int codes kept as raw bits for TableAt
  float start[CPL];     // approximate prefix sum in front of each chunk
  float approx_total;
  {
    float pre[CPL + 1];
    pre[0] = 0.0f;
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const int k = lane * CPL + c;
      pre[c + 1] = pre[c] + (k < NCH ? lds->approx[k] : 0.0f);
    }
    const float incl = WaveInclusiveScanF32(pre[CPL]);
    const float excl = incl - pre[CPL];
    approx_total = ReadLaneF32(incl, kWave - 1);
    int raw[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      start[c] = excl + pre[c];
      raw[c] = PlanPiece(start[c], excl + pre[c + 1], margin);
    }
    /* neighbouring clean chunks must agree on the binade, or the later one is walked:
       every run of clean chunks then has one scale */
    const int before = __shfl_up(raw[CPL - 1], 1);
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const int prev = (c == 0) ? ((lane == 0) ? kPlanWalk : before) : raw[c - 1];
      const bool clash = IsClean(raw[c]) && IsClean(prev) && prev != raw[c];
      code[c] = static_cast<uint32_t>(clash ? kPlanTwoBinades + (prev < raw[c] ? prev : raw[c]) : raw[c]);
    }
  }
  /* a NaN among the terms makes the sum NaN whatever the order */
  if (approx_total != approx_total) return approx_total;

  /* C: integer totals of this wave's clean chunks ... */
  MSHADOW_ROWSUM_STAMP(2)
  uint32_t dirty_mask;  // this wave's slabs that have to be walked
  uint32_t tie_mask;    // of those, planned clean but found to hold a tie
  {
    float part[SLABS];
#pragma unroll
    for (int j = 0; j < SLABS; ++j) {
      const int k = wave * SLABS + j;
      const int ck = static_cast<int>(ReadLaneU32(code[j % CPL], k / CPL));
      part[j] = 0.0f;
      if (IsClean(ck)) part[j] = LaneQuant<N>(v[j], BinadeOfExponent(static_cast<uint32_t>(ck)));
    }
    const float q = mshadow::hip::WaveSumMany<SLABS>(part);  // lane l: chunk l % SLABS
    /* lanes 0 .. SLABS-1 file the result of "their" chunk; its plan code sits in the
       chunk table at lane k / CPL, slot k % CPL = lane % CPL */
    const int k = wave * SLABS + (lane % SLABS);
    int ck = 0;
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const int got = __shfl(static_cast<int>(code[c]), k / CPL);
      ck = (lane % CPL == c) ? got : ck;
    }
    const bool clean = IsClean(ck);
    const bool whole = clean && q < kLimit;  // a tie anywhere in the chunk pushes q past 2^24
    if (lane < SLABS) {
      lds->q[k] = whole ? static_cast<uint32_t>(q) : kDirtyQ;
    }
    dirty_mask = static_cast<uint32_t>(__ballot(lane < SLABS && !whole));
    tie_mask = static_cast<uint32_t>(__ballot(lane < SLABS && clean && !whole));
  }
  /* ... and its dirty ones handed, with their terms, to plan slots: the lane plans are
     made by all waves together further down (the first wave of a row owns most dirty chunks) */
  for (uint32_t todo = dirty_mask; todo != 0u; todo &= todo - 1u) {
    const int j = __ffs(static_cast<int>(todo)) - 1;
    const int k = wave * SLABS + j;
    uint32_t slot = 0u;
    if (lane == 0) slot = atomicAdd(&lds->nslots, 1u);
    slot = __builtin_amdgcn_readfirstlane(slot);
    if (slot >= static_cast<uint32_t>(Lds::kSlots)) {  // no room: the row is redone by wave scans
      if (lane == 0) lds->fail = 1;
      break;
    }
    float t[N];
    SelectSlab<SLABS, N>(t, v, j);
    LanePlanSlot<N> *ps = &lds->plan[slot];
#pragma unroll
    for (int i = 0; i < N; ++i) ps->t[lane][i] = t[i];
    int ck = static_cast<int>(TableAt<CPL>(code, k));
    if ((tie_mask >> j) & 1u) ck = kPlanTwoBinades + ck;
    uint32_t start_bits[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) start_bits[c] = __float_as_uint(start[c]);
    const float st = __uint_as_float(TableAt<CPL>(start_bits, k));
    if (lane == 0) {
      ps->kind = ck;
      ps->start = st;
      ps->chunk = k;
    }
  }
  __syncthreads();
  MSHADOW_ROWSUM_STAMP(3)
  /* D: tables of the walk */
  uint32_t ex[CPL];  // integer prefix over clean chunks in front of each chunk
  uint32_t total_ex;
  {
    uint32_t pre[CPL + 1];
    pre[0] = 0u;
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const int k = lane * CPL + c;
      const uint32_t q = k < NCH ? lds->q[k] : 0u;
      if (q == kDirtyQ && IsClean(static_cast<int>(code[c]))) code[c] = static_cast<uint32_t>(kPlanWalk);
      const bool is_dirty = k < NCH && !IsClean(static_cast<int>(code[c]));
      pre[c + 1] = pre[c] + (is_dirty ? 0u : q);
    }
    const uint32_t incl = WaveInclusiveScanU32(pre[CPL]);
    const uint32_t excl = incl - pre[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) ex[c] = excl + pre[c];
    total_ex = ReadLaneU32(incl, kWave - 1);
  }
  /* lane plans of the dirty chunks, made by all waves together */
  {
    const uint32_t handed = lds->nslots;
    const int nslots = handed < static_cast<uint32_t>(Lds::kSlots) ? static_cast<int>(handed) : Lds::kSlots;
    /* slots were handed out in no particular order: the walk takes them by chunk number */
    const int chunk_of_lane = lane < nslots ? lds->plan[lane < Lds::kSlots ? lane : 0].chunk : 0x7fffffff;
    for (int sl = wave; sl < nslots; sl += W) {
      LanePlanSlot<N> *ps = &lds->plan[sl];
      float t[N];
#pragma unroll
      for (int i = 0; i < N; ++i) t[i] = ps->t[lane][i];
      const int ck = ps->kind;
      uint32_t pa, pb;
      if (ck >= kPlanTwoBinades) {
        unsigned long long tlo, thi;
        PlanTwoBinades<N>(t, ck - kPlanTwoBinades, &pa, &pb, &tlo, &thi);
        if (lane == 0) {
          ps->tie_lo = tlo;
          ps->tie_hi = thi;
        }
      } else {
        int code_l;
        const uint32_t tot = PlanLanes<N>(t, ps->start, margin, ps->chunk == 0, &pa, &code_l);
        pb = static_cast<uint32_t>(code_l);
        if (lane == 0) ps->total = tot;
      }
      ps->a[lane] = pa;
      ps->b[lane] = pb;
      /* what the walk needs from the chunk table, so that it reads scalars only */
      const int k = ps->chunk;
      const uint32_t exk = TableAt<CPL>(ex, k);
      const uint32_t erun = k > 0 ? TableAt<CPL>(code, k - 1) : 0u;
      const int rank = __popcll(__ballot(chunk_of_lane < k));
      if (lane == 0) {
        ps->ex = exk;
        ps->e_run = static_cast<int>(erun);
        lds->order[rank] = static_cast<signed char>(sl);
      }
    }
  }

  __syncthreads();
  MSHADOW_ROWSUM_STAMP(4)
  /* the walk: one wave takes the dirty chunks in row order; everything it needs sits in the
     plan slots */
  if (wave == 0 && lds->fail == 0) {
    MSHADOW_ROWSUM_STAMP(8)
    /* the whole row waits for this chain; the other waves on this SIMD (another row's bulk
       phases) yield issue slots to it */
    __builtin_amdgcn_s_setprio(3);
    const uint32_t handed = lds->nslots;
    const int nslots = handed < static_cast<uint32_t>(Lds::kSlots) ? static_cast<int>(handed) : Lds::kSlots;
    const int slot_at = lane < nslots ? lds->order[lane < Lds::kSlots ? lane : 0] : 0;
    float s = 0.0f;
    uint32_t done = 0u;
    bool fail = false;
    /* the lane-wise part of the next chunk's slot is fetched while the current chunk's chain
       of dependent instructions runs (none of it depends on the running sum) */
    float nt[N];
    uint32_t npa = 0u, npb = 0u;
    const LanePlanSlot<N> *nps = &lds->plan[ReadLaneU32(static_cast<uint32_t>(slot_at), 0)];
    if (nslots > 0) {
#pragma unroll
      for (int e = 0; e < N; ++e) nt[e] = nps->t[lane][e];
      npa = nps->a[lane];
      npb = nps->b[lane];
    }
    for (int i = 0; i < nslots; ++i) {
      const LanePlanSlot<N> *ps = nps;
      float t[N];
#pragma unroll
      for (int e = 0; e < N; ++e) t[e] = nt[e];
      const uint32_t pa = npa, pb = npb;
      const int kind = ps->kind;
      const uint32_t exk = ps->ex;
      const int erun = ps->e_run;
      if (i + 1 < nslots) {
        nps = &lds->plan[ReadLaneU32(static_cast<uint32_t>(slot_at), i + 1)];
#pragma unroll
        for (int e = 0; e < N; ++e) nt[e] = nps->t[lane][e];
        npa = nps->a[lane];
        npb = nps->b[lane];
      }
      if (exk != done) {
        s = FlushRun(s, erun, exk - done, &fail);
        done = exk;
      }
      if (kind >= kPlanTwoBinades) {
        s = WalkTwoBinades<N>(s, t, kind - kPlanTwoBinades, pa, pb, ps->tie_lo, ps->tie_hi, &fail);
      } else if (ps->chunk == 0) {
        s = HeadSerialAdd<N>(s, ps->t);
        s = WalkLanes<N>(s, t, pa, static_cast<int>(pb), ps->total, (1ull << kHeadLanes) - 1ull, &fail);
      } else {
        s = WalkLanes<N>(s, t, pa, static_cast<int>(pb), ps->total, 0ull, &fail);
      }
    }
    if (lane == 0) {
      lds->s = s;
      lds->ex = done;
      if (fail) lds->fail = 1;
    }
    __builtin_amdgcn_s_setprio(0);
    MSHADOW_ROWSUM_STAMP(9)
  }
  __syncthreads();

  /* E: the clean run behind the last dirty chunk */
  MSHADOW_ROWSUM_STAMP(5)
  float s = lds->s;
  bool fail = lds->fail != 0;
  if (total_ex != lds->ex) {
    s = FlushRun(s, static_cast<int>(TableAt<CPL>(code, NCH - 1)), total_ex - lds->ex, &fail);
  }
  MSHADOW_ROWSUM_STAMP(6)
  if (!fail) return s;
  MSHADOW_ROWSUM_STAMP(7)

  /* a plan did not hold (kept so that the result cannot depend on the plan): every chunk
     is resolved in order by wave scans, wave after wave */
  __syncthreads();
  if (threadIdx.x == 0) lds->s = 0.0f;
  __syncthreads();
  for (int w = 0; w < W; ++w) {
    if (wave == w) {
      float r = lds->s;
      for (int j = 0; j < SLABS; ++j) {
        float t[N];
        SelectSlab<SLABS, N>(t, v, j);
        r = WaveResolve<N>(r, t);
      }
      if (lane == 0) lds->s = r;
    }
    __syncthreads();
  }
  return lds->s;
}

/*! \brief e^x for x <= 0 (any float accepted): 2^(x * log2 e) with the rounding error of
 *  the product carried separately, so the result stays within about 1.5 ulp for the whole
 *  range a softmax sees. The hardware exp2 does not return subnormals, so results below
 *  2^-126 are computed 64 binades up and scaled back. */
__device__ __forceinline__ float ExpNonPositive(float x) {
  const float kLog2eHi = 1.44269502162933349609375f;
  const float kLog2eLo = 1.925963033500011079013347625732421875e-08f;
  const float t = x * kLog2eHi;
  float r = __builtin_fmaf(x, kLog2eHi, -t);   // exact rounding error of the product
  r = __builtin_fmaf(x, kLog2eLo, r);
  if (__builtin_expect(!(t >= -125.0f), 0)) {   // subnormal / zero result, -inf, NaN
    if (t < -151.0f) return 0.0f;               // below half of the smallest subnormal
    const float e = __builtin_amdgcn_exp2f(t + 64.0f);
    const float v = __builtin_fmaf(e, r * 0.693147182464599609375f, e);
    return v * 5.42101086242752217003726400434970855712890625e-20f;  // 2^-64
  }
  const float e = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(e, r * 0.693147182464599609375f, e);  // e * 2^r, |r| << 1
}

/*! \brief p / s given rcp = 1 / s: one Newton correction on the quotient. The result is
 *  the correctly rounded quotient except for rare half-ulp cases. */
__device__ __forceinline__ float DivideBy(float p, float s, float rcp) {
  const float q = p * rcp;
  const float e = __builtin_fmaf(-q, s, p);
  return __builtin_fmaf(e, rcp, q);
}

template <int THREADS>
__device__ inline float BlockMax(float v, float *wmax) {
  const int W = THREADS / kWave;
  v = WaveMaxF32(v);
  if (LaneId() == 0) wmax[WaveId()] = v;
  __syncthreads();
  float m = wmax[0];
#pragma unroll
  for (int w = 1; w < W; ++w) {
    const float o = wmax[w];
    m = (m < o) ? o : m;
  }
  return m;
}

/*! \brief THREADS * SLABS * VEC >= cols. VEC == 4 needs 16-byte aligned rows and
 *  cols % 4 == 0. Wave w holds columns [w, w + 1) * SLABS * 64 * VEC, slab j of it the
 *  next 64 * VEC, lane l of that VEC consecutive ones: each load is one contiguous
 *  kilobyte per wave and the order of the row is wave, slab, lane, element.
 *  TERMS_GIVEN: src already holds the (non-negative) terms and dst[row] receives their
 *  left-to-right sum - the row-sum stage on its own. */
template <int THREADS, int SLABS, int VEC, bool TERMS_GIVEN>
__global__ void __launch_bounds__(THREADS, 4)  // >= 4 waves per SIMD: two 512-thread rows per CU
    SoftmaxRowKernel(float *dst, int dstride, const float *src, int sstride, int cols) {
  __shared__ RowSumLds<THREADS / kWave, SLABS, VEC> lds;
  const int wave = __builtin_amdgcn_readfirstlane(WaveId());
  const int lane = LaneId();
  const float *in = src + static_cast<size_t>(blockIdx.x) * sstride;
  float *out = dst + static_cast<size_t>(blockIdx.x) * dstride;
  const float kNegInf = -__builtin_huge_valf();
  const float kAbsent = TERMS_GIVEN ? 0.0f : kNegInf;

  float v[SLABS][VEC];
  float mx = kNegInf;
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int base = ((wave * SLABS + j) * kWave + lane) * VEC;
    if (VEC == 4) {  // cols % 4 == 0: a pack is either whole or absent
      F4 q = {kAbsent, kAbsent, kAbsent, kAbsent};
      if (base < cols) q = StreamLoadF4(in + base);
      v[j][0] = q.x; v[j][1 % VEC] = q.y; v[j][2 % VEC] = q.z; v[j][3 % VEC] = q.w;
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[j][i] = (base + i < cols) ? in[base + i] : kAbsent;
    }
    if (!TERMS_GIVEN) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) mx = (mx < v[j][i]) ? v[j][i] : mx;
    }
  }
  if (!TERMS_GIVEN) {
    mx = BlockMax<THREADS>(mx, lds.wmax);
#pragma unroll
    for (int j = 0; j < SLABS; ++j) {
      const int base = ((wave * SLABS + j) * kWave + lane) * VEC;
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[j][i] = (base + i < cols) ? ExpNonPositive(v[j][i] - mx) : 0.0f;
    }
  }

  const float s = RowOrderedSum<THREADS, SLABS, VEC>(v, cols, &lds);
  if (TERMS_GIVEN) {
    if (threadIdx.x == 0) dst[blockIdx.x] = s;
    return;
  }

  /* s >= 1 for finite logits (the maximum contributes exp(0)); anything else (NaN or
     infinite logits) takes the plain division so that specials propagate as on the CPU */
  const bool fast_div = s >= 1.0f && s < 3.0e38f;
  const float rcp = 1.0f / s;
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int base = ((wave * SLABS + j) * kWave + lane) * VEC;
    float o[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) o[i] = fast_div ? DivideBy(v[j][i], s, rcp) : v[j][i] / s;
    if (VEC == 4) {
      F4 q;
      q.x = o[0]; q.y = o[1 % VEC]; q.z = o[2 % VEC]; q.w = o[3 % VEC];
      if (base < cols) StreamStoreF4(out + base, q);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        if (base + i < cols) out[base + i] = o[i];
      }
    }
  }
}

/* ---- short rows -----------------------------------------------------------------------
 * A workgroup per row wastes the machine on the rows classifiers usually have (tens to a few
 * hundred classes). Same arithmetic as SoftmaxRowKernel, other ownership: */

/*! \brief one thread per row, cols <= CMAX: the row sits in the thread's registers and its
 *  sum is the serial loop itself. A wave reads 64 neighbouring rows, so the cache lines it
 *  touches are used whole. */
template <int CMAX, bool TERMS_GIVEN>
__global__ void __launch_bounds__(256)
    SoftmaxThreadRowKernel(float *dst, int dstride, const float *src, int sstride, int rows,
                           int cols) {
  const int row = blockIdx.x * 256 + threadIdx.x;
  if (row >= rows) return;
  const float *in = src + static_cast<size_t>(row) * sstride;
  const float kNegInf = -__builtin_huge_valf();
  float v[CMAX];
  float mx = kNegInf;
#pragma unroll
  for (int i = 0; i < CMAX; ++i) {
    v[i] = (i < cols) ? in[i] : (TERMS_GIVEN ? 0.0f : kNegInf);
    mx = (mx < v[i]) ? v[i] : mx;
  }
  if (!TERMS_GIVEN) {
#pragma unroll
    for (int i = 0; i < CMAX; ++i) v[i] = (i < cols) ? ExpNonPositive(v[i] - mx) : 0.0f;
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < CMAX; ++i) {
    if (i < cols) s = s + v[i];
  }
  if (TERMS_GIVEN) {
    dst[row] = s;
    return;
  }
  float *out = dst + static_cast<size_t>(row) * dstride;
  const bool fast_div = s >= 1.0f && s < 3.0e38f;
  const float rcp = 1.0f / s;
#pragma unroll
  for (int i = 0; i < CMAX; ++i) {
    if (i < cols) out[i] = fast_div ? DivideBy(v[i], s, rcp) : v[i] / s;
  }
}

/*! \brief one wave per row, cols <= 64 * N: lane l holds the N consecutive columns from
 *  l * N, the sum is resolved in lane order by wave scans (WaveResolve), four rows per
 *  workgroup and nothing shared between them */
template <int N, bool TERMS_GIVEN>
__global__ void __launch_bounds__(256)
    SoftmaxWaveRowKernel(float *dst, int dstride, const float *src, int sstride, int rows,
                         int cols) {
  const int row = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(WaveId());
  if (row >= rows) return;
  const int base = LaneId() * N;
  const float *in = src + static_cast<size_t>(row) * sstride;
  const float kNegInf = -__builtin_huge_valf();
  float v[N];
  float mx = kNegInf;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    v[i] = (base + i < cols) ? in[base + i] : (TERMS_GIVEN ? 0.0f : kNegInf);
    mx = (mx < v[i]) ? v[i] : mx;
  }
  if (!TERMS_GIVEN) {
    mx = WaveMaxF32(mx);
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = (base + i < cols) ? ExpNonPositive(v[i] - mx) : 0.0f;
  }
  const float s = WaveResolve<N>(0.0f, v);
  if (TERMS_GIVEN) {
    if (LaneId() == 0) dst[row] = s;
    return;
  }
  float *out = dst + static_cast<size_t>(row) * dstride;
  const bool fast_div = s >= 1.0f && s < 3.0e38f;
  const float rcp = 1.0f / s;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if (base + i < cols) out[base + i] = fast_div ? DivideBy(v[i], s, rcp) : v[i] / s;
  }
}

/*! \brief any row length: three passes, exp(x - max) parked in dst between them */
template <int THREADS>
__global__ void __launch_bounds__(THREADS)
    SoftmaxLongRowKernel(float *dst, int dstride, const float *src, int sstride, int cols) {
  __shared__ OrderedSumLds<THREADS / kWave> lds;
  const int tid = threadIdx.x;
  const float *in = src + static_cast<size_t>(blockIdx.x) * sstride;
  float *out = dst + static_cast<size_t>(blockIdx.x) * dstride;
  const float kNegInf = -__builtin_huge_valf();
  float mx = kNegInf;
  for (int x = tid; x < cols; x += THREADS) {
    const float e = in[x];
    mx = (mx < e) ? e : mx;
  }
  mx = BlockMax<THREADS>(mx, lds.wmax);
  float s = 0.0f;
  int buf = 0;
  for (int x0 = 0; x0 < cols; x0 += THREADS) {
    const int x = x0 + tid;
    float p[1];
    p[0] = (x < cols) ? ExpNonPositive(in[x] - mx) : 0.0f;
    if (x < cols) out[x] = p[0];
    s = BlockOrderedAdd<THREADS, 1>(s, p, &lds, &buf);
  }
  for (int x = tid; x < cols; x += THREADS) out[x] = out[x] / s;
}

const int kGradBlock = 256;
const int kGradPacks = 1;  // 128-bit packs per thread

/*! \brief flags of the gradient family (mshadow/tensor_cpu-inl.h:287-462) */
const int kGradSmooth = 1;  //!< SmoothSoftmaxGrad: alpha is spread over the other classes
const int kGradIgnore = 2;  //!< rows whose label equals ignore_label get a zero gradient

struct GradParams {
  int ignore_label;   //!< static_cast<int>(ignore_label)
  float alpha;
  float smooth_grad;  //!< alpha / (classes - 1), computed in float like the reference
};

/*! \brief one element of the gradient; the expressions are the reference's, in its order */
template <int FLAGS>
__device__ __forceinline__ float GradElement(float s, bool at_label, bool ignored, const GradParams &p) {
  float v;
  if (at_label) {
    v = s - 1.0f;
    if (FLAGS & kGradSmooth) v = v + p.alpha;
  } else {
    v = s;
    if (FLAGS & kGradSmooth) v = v - p.smooth_grad;
  }
  if ((FLAGS & kGradIgnore) && ignored) v = 0.0f;
  return v;
}

/*! \brief grid.x = rows * chunks, a chunk being kGradBlock * kGradPacks * 4 columns.
 *  Consecutive workgroups walk along a row, so the workgroups in flight at any moment
 *  stream one contiguous region of memory. */
template <bool VEC4, int FLAGS>
__global__ void __launch_bounds__(kGradBlock)
    SoftmaxGradKernel(float *dst, int dstride, const float *src, int sstride, const float *label,
                      int cols, unsigned chunks, GradParams gp) {
  const int y = blockIdx.x / chunks;
  const int chunk = blockIdx.x - y * chunks;
  const int k = static_cast<int>(label[y]);
  const bool ignored = (FLAGS & kGradIgnore) && k == gp.ignore_label;
  const float *in = src + static_cast<size_t>(y) * sstride;
  float *out = dst + static_cast<size_t>(y) * dstride;
  const int chunk0 = chunk * (kGradBlock * kGradPacks * 4);
  if (VEC4) {
    F4 q[kGradPacks];
#pragma unroll
    for (int u = 0; u < kGradPacks; ++u) {
      const int x = chunk0 + (u * kGradBlock + threadIdx.x) * 4;
      if (x + 4 <= cols) q[u] = StreamLoadF4(in + x);
    }
#pragma unroll
    for (int u = 0; u < kGradPacks; ++u) {
      const int x = chunk0 + (u * kGradBlock + threadIdx.x) * 4;
      if (x + 4 <= cols) {
        if (FLAGS == 0) {
          if (k == x) q[u].x = q[u].x - 1.0f;
          if (k == x + 1) q[u].y = q[u].y - 1.0f;
          if (k == x + 2) q[u].z = q[u].z - 1.0f;
          if (k == x + 3) q[u].w = q[u].w - 1.0f;
        } else {
          q[u].x = GradElement<FLAGS>(q[u].x, k == x, ignored, gp);
          q[u].y = GradElement<FLAGS>(q[u].y, k == x + 1, ignored, gp);
          q[u].z = GradElement<FLAGS>(q[u].z, k == x + 2, ignored, gp);
          q[u].w = GradElement<FLAGS>(q[u].w, k == x + 3, ignored, gp);
        }
        StreamStoreF4(out + x, q[u]);
      } else {
        for (int i = x; i < cols; ++i) out[i] = GradElement<FLAGS>(in[i], i == k, ignored, gp);
      }
    }
  } else {
#pragma unroll
    for (int u = 0; u < kGradPacks * 4; ++u) {
      const int x = chunk0 + u * kGradBlock + threadIdx.x;
      if (x < cols) out[x] = GradElement<FLAGS>(in[x], x == k, ignored, gp);
    }
  }
}

/* ---- 3-D tensors (d0, d1, d2), softmax over d1, row pitch on d2 ----------------------
 * (mshadow/tensor_cpu-inl.h:474-495; cuda/tensor_gpu-inl.cuh:479-597). One thread per
 * (y, n) pair, n fastest: every access of a wave is one contiguous run along d2, and the
 * max / sum over the classes is a serial loop in the thread - the reference's own order. */
const int kSoftmax3dBlock = 256;

__global__ void __launch_bounds__(kSoftmax3dBlock)
    Softmax3dKernel(float *dst, int dstride, const float *src, int sstride, int d0, int d1, int d2,
                    mshadow::FastDivU32 div_d2) {
  const unsigned total = static_cast<unsigned>(d0) * d2;
  for (unsigned i = blockIdx.x * kSoftmax3dBlock + threadIdx.x; i < total;
       i += gridDim.x * kSoftmax3dBlock) {
    const unsigned y = div_d2.Div(i);
    const unsigned n = i - y * d2;
    const float *in = src + static_cast<size_t>(y) * d1 * sstride + n;
    float *out = dst + static_cast<size_t>(y) * d1 * dstride + n;
    float mx = in[0];
    for (int x = 1; x < d1; ++x) {
      const float e = in[static_cast<size_t>(x) * sstride];
      mx = (mx < e) ? e : mx;
    }
    float sum = 0.0f;
    for (int x = 0; x < d1; ++x) {
      const float p = ExpNonPositive(in[static_cast<size_t>(x) * sstride] - mx);
      out[static_cast<size_t>(x) * dstride] = p;
      sum = sum + p;
    }
    const bool fast_div = sum >= 1.0f && sum < 3.0e38f;
    const float rcp = 1.0f / sum;
    for (int x = 0; x < d1; ++x) {
      const float p = out[static_cast<size_t>(x) * dstride];
      out[static_cast<size_t>(x) * dstride] = fast_div ? DivideBy(p, sum, rcp) : p / sum;
    }
  }
}

/*! \brief the same for at most D1MAX classes: the column of one (y, n) pair is fetched once
 *  (all loads in flight together), kept in registers and written once */
template <int D1MAX>
__global__ void __launch_bounds__(kSoftmax3dBlock)
    Softmax3dSmallKernel(float *dst, int dstride, const float *src, int sstride, int d0, int d1,
                         int d2, mshadow::FastDivU32 div_d2) {
  const unsigned total = static_cast<unsigned>(d0) * d2;
  const unsigned i = blockIdx.x * kSoftmax3dBlock + threadIdx.x;
  if (i >= total) return;
  const unsigned y = div_d2.Div(i);
  const unsigned n = i - y * d2;
  const float *in = src + static_cast<size_t>(y) * d1 * sstride + n;
  float *out = dst + static_cast<size_t>(y) * d1 * dstride + n;
  float v[D1MAX];
#pragma unroll
  for (int x = 0; x < D1MAX; ++x) {
    /* unpredicated: classes past the end re-read the last one and are not used */
    v[x] = StreamLoad(in + static_cast<size_t>(x < d1 ? x : d1 - 1) * sstride);
  }
  float mx = v[0];
#pragma unroll
  for (int x = 1; x < D1MAX; ++x) {
    if (x < d1) mx = (mx < v[x]) ? v[x] : mx;
  }
  float sum = 0.0f;
#pragma unroll
  for (int x = 0; x < D1MAX; ++x) {
    if (x < d1) {
      v[x] = ExpNonPositive(v[x] - mx);
      sum = sum + v[x];
    }
  }
  const bool fast_div = sum >= 1.0f && sum < 3.0e38f;
  const float rcp = 1.0f / sum;
#pragma unroll
  for (int x = 0; x < D1MAX; ++x) {
    if (x < d1) {
      StreamStore(out + static_cast<size_t>(x) * dstride, fast_div ? DivideBy(v[x], sum, rcp) : v[x] / sum);
    }
  }
}

/*! \brief gradient on 3-D tensors: label is (d0, d2) with pitch lstride; elementwise over
 *  the (d0 * d1, d2) view, VEC consecutive n per thread (VEC = 4 needs d2 % 4 == 0 and
 *  16-byte aligned rows) */
template <int FLAGS>
__global__ void __launch_bounds__(kSoftmax3dBlock)
    Softmax3dGradVecKernel(float *dst, int dstride, const float *src, int sstride,
                           const float *label, int lstride, int d0, int d1, int d2,
                           mshadow::FastDivU32 div_q2, mshadow::FastDivU32 div_d1, GradParams gp) {
  const unsigned q2 = static_cast<unsigned>(d2) / 4;  // packs per row
  const unsigned total = static_cast<unsigned>(d0) * d1 * q2;
  const unsigned i = blockIdx.x * kSoftmax3dBlock + threadIdx.x;
  if (i >= total) return;
  const unsigned row = div_q2.Div(i);
  const unsigned n = (i - row * q2) * 4;
  const unsigned y = div_d1.Div(row);
  const int x = static_cast<int>(row - y * d1);
  const F4 l = *reinterpret_cast<const F4 *>(label + static_cast<size_t>(y) * lstride + n);
  F4 s = StreamLoadF4(src + static_cast<size_t>(row) * sstride + n);
  const int k0 = static_cast<int>(l.x), k1 = static_cast<int>(l.y), k2 = static_cast<int>(l.z),
            k3 = static_cast<int>(l.w);
  s.x = GradElement<FLAGS>(s.x, x == k0, (FLAGS & kGradIgnore) && k0 == gp.ignore_label, gp);
  s.y = GradElement<FLAGS>(s.y, x == k1, (FLAGS & kGradIgnore) && k1 == gp.ignore_label, gp);
  s.z = GradElement<FLAGS>(s.z, x == k2, (FLAGS & kGradIgnore) && k2 == gp.ignore_label, gp);
  s.w = GradElement<FLAGS>(s.w, x == k3, (FLAGS & kGradIgnore) && k3 == gp.ignore_label, gp);
  StreamStoreF4(dst + static_cast<size_t>(row) * dstride + n, s);
}

/*! \brief any alignment: one element per thread-iteration */
template <int FLAGS>
__global__ void __launch_bounds__(kSoftmax3dBlock)
    Softmax3dGradKernel(float *dst, int dstride, const float *src, int sstride, const float *label,
                        int lstride, int d0, int d1, int d2, mshadow::FastDivU32 div_d2,
                        mshadow::FastDivU32 div_d1, GradParams gp) {
  const unsigned total = static_cast<unsigned>(d0) * d1 * d2;
  for (unsigned i = blockIdx.x * kSoftmax3dBlock + threadIdx.x; i < total;
       i += gridDim.x * kSoftmax3dBlock) {
    const unsigned row = div_d2.Div(i);       // y * d1 + x
    const unsigned n = i - row * d2;
    const unsigned y = div_d1.Div(row);
    const int x = static_cast<int>(row - y * d1);
    const int k = static_cast<int>(label[static_cast<size_t>(y) * lstride + n]);
    const float s = src[static_cast<size_t>(row) * sstride + n];
    dst[static_cast<size_t>(row) * dstride + n] =
        GradElement<FLAGS>(s, x == k, (FLAGS & kGradIgnore) && k == gp.ignore_label, gp);
  }
}

}  // namespace mshadow_hipk
#endif  // MSHADOW_AMD_CSRC_SOFTMAX_KERNELS_H_
