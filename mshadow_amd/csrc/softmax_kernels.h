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
 * SoftmaxStretchRowKernel covers rows too long for registers with the same arithmetic,
 * stretch by stretch. SoftmaxGradKernel is a 128-bit copy with one element per row
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

/*! \brief the larger of two / three floats, a NaN operand ignored (one instruction; the
 *  source-level forms compile to a compare and a select, or to extra canonicalising ops) */
__device__ __forceinline__ float MaxNum(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float MaxNum3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

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

/* ---- planned row sum (registers hold the whole row) ---------------------------------
 * Thread layout: chunk k of the row (64 * N consecutive terms, lane-major) is slab k / W of
 * wave k % W, so the W waves walk the row side by side and the chunks next to the row's
 * binade crossings are spread over the waves. ordered_sum.h describes the plan; the steps are
 *   A  every wave: approximate sum and largest term of each of its chunks -> LDS   (barrier)
 *   B  every wave (redundantly): prefix over all chunks, a binade per chunk where certain
 *   C  every wave: its certain chunks quantised against their binade, integer totals -> LDS;
 *      each of its other chunks planned lane by lane and written to LDS as a short list
 *      of addends (a run of certain lanes = one addend, any other lane = its terms) (barrier)
 *   D  every wave (redundantly): integer prefix over the certain chunks, the place of every
 *      list in the row's list of addends; the lists are copied there, each by one wave, with
 *      the run of certain chunks in front of each listed chunk as one more addend  (barrier)
 *   E  wave 0: the chain - the row's addends summed serially, every run verified  (barrier)
 * A row whose plan fails a verification, or that has more listed chunks than slots, is summed
 * by wave scans instead, chunk after chunk. The sum may start from s0 instead of zero (a row
 * longer than the registers hold is summed stretch by stretch): s0 then stands in front of the
 * approximate prefix sums and is where the chain begins.
 * Lane l keeps the chunk-table entries of chunks l * CPL .. l * CPL + CPL - 1. */
/*! \brief chunks per row that can hand a list of addends to the chain (a row of softmax
 *  terms has about a dozen) */
const int kPlanSlots = 24;
const uint32_t kListedBit = 0x80000000u;

/* hook for a profiling build: a translation unit may define this to record a timestamp
   at the boundaries of the steps; it is empty in the library */
#ifndef MSHADOW_ROWSUM_STAMP
#define MSHADOW_ROWSUM_STAMP(step)
#endif


/*! \brief one addend of the chain: its value and, for a run, 1 + the binade the sum must be
 *  in before and after it (0 for a term); eight bytes, written and read as one word */
struct Addend {
  float value;
  uint32_t check;
};
/*! \brief the addends of one listed chunk, in row order: at most one per term */
template <int N>
struct AddendList {
  Addend entry[kWave * N];
};

template <int W, int SLABS, int N>
struct RowSumLds {
  static const int kChunks = W * SLABS;
  /* small workgroups share a CU with several others: fewer slots each */
  static const int kWanted = W <= 4 ? kPlanSlots * 2 / 3 : kPlanSlots;
  static const int kSlots = (kChunks < kWanted) ? kChunks : kWanted;
  float approx[kChunks];
  float cmax[kChunks];
  /*! \brief what a listed chunk's wave needs of the plan. Every wave computes the whole
   *  plan and files it here (the same values from each), then reads its own chunks' entries
   *  back: a wave sees its own stores, so no barrier is involved. */
  struct ChunkPlan {
    float start;    //!< approximate prefix sum in front of the chunk
    float low;      //!< what the sum is at least in front of the chunk
    uint32_t slot;  //!< the chunk's slot, if the plan lists it
    uint32_t peak;  //!< the chunk holds a term above `low` (it can raise the bound inside the chunk)
  };
  MSHADOW_ALIGNED(16) ChunkPlan plan[kChunks];
  /*! \brief certain chunk: its integer total; listed chunk: kListedBit | addends << 8 | slot */
  uint32_t q[kChunks];
  float s;          //!< the row's sum, from the chain to everybody
  int fail;         //!< the plan did not hold: redo the row the slow way
  uint32_t nslots;  //!< lists handed out
  float wmax[W];
  /*! \brief the row's addends in row order, as the chain takes them: for each listed chunk
   *  the run of certain chunks in front of it (one addend) and then its own list, and
   *  at the end the run behind the last listed chunk */
  /* 512 hold nearly every row; a row whose sum ends just above a power of two has every chunk
     behind the crossing listed lane by lane (the bounds cannot tell on which side the sum is)
     and takes 900-1100, so workgroups of eight waves and more, two to a CU, have room for 2048:
     the chain over them is a few microseconds, the fall-back 45 */
  static const int kRowAddends = W <= 4 ? 512 : 2048;
  Addend row[kRowAddends];
  uint32_t row_count;
  MSHADOW_ALIGNED(8) AddendList<N> list[kSlots];
};

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

/*! \brief value of v in the lane below (lane 0 receives `first`) */
__device__ __forceinline__ uint32_t FromLaneBelowU32(uint32_t v, uint32_t first) {
  /* DPP wave_shr:1; a lane without a source keeps the first operand */
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(first), static_cast<int>(v),
                                                           0x138, 0xf, 0xf, false));
}

/*! \brief one step of the serial sum that runs along the lanes of a wave: lane l takes
 *  the sum of lane l - 1 and adds its own addend; lane 0 has no lane below it and keeps its
 *  value. After k steps lanes 0 .. k hold the sums after their addends, for good (a lane's
 *  value depends only on the settled lane below it), so surplus steps change nothing. One
 *  VALU instruction on the dependent path; the idle cycles in front of it are what the
 *  hardware asks for between writing a register and reading it through DPP. */
__device__ __forceinline__ void SystolicStep(float *sum, float addend) {
  asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %0, %1 wave_shr:1 row_mask:0xf bank_mask:0xf"
               : "+v"(*sum)
               : "v"(addend));
}

/*! \brief eight such steps */
__device__ __forceinline__ void SystolicSteps8(float *sum, float addend) {
#define MSHADOW_STEP "s_nop 1\n\tv_add_f32_dpp %0, %0, %1 wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
  asm volatile(MSHADOW_STEP MSHADOW_STEP MSHADOW_STEP MSHADOW_STEP MSHADOW_STEP MSHADOW_STEP
                   MSHADOW_STEP MSHADOW_STEP "s_nop 1"
               : "+v"(*sum)
               : "v"(addend));
#undef MSHADOW_STEP
}

/*! \brief s plus up to 64 addends, lane l holding addend l (`count` of them, zeros behind),
 *  one float add after the other; check = 1 + binade for a run (0 for a term). A lane whose
 *  run was added while the sum was not in its binade sets its *bad. */
__device__ __forceinline__ float ChainBlock(float s, float addend, uint32_t check, int count,
                                            bool *bad) {
  using namespace ordered_sum;
  float sum = s + addend;  // right in lane 0, the start of the systolic sum
  for (int done = 1; done < count; done += 8) SystolicSteps8(&sum, addend);
  const float before = __uint_as_float(FromLaneBelowU32(__float_as_uint(sum), __float_as_uint(s)));
  *bad = *bad || (check != 0u && !RunHolds(before, sum, check - 1u));
  return ReadLaneF32(sum, count - 1);
}

template <int THREADS, int SLABS, int N, bool CHECK_SIGN, bool UNIT_PEAK>
__device__ inline float RowOrderedSum(const float (&v)[SLABS][N], int cols,
                                      RowSumLds<THREADS / kWave, SLABS, N> *lds, float s0 = 0.0f) {
  using namespace ordered_sum;
  using mshadow::hip::ReadLaneU32;
  using mshadow::hip::WaveInclusiveScanU32;
  typedef RowSumLds<THREADS / kWave, SLABS, N> Lds;
  const int W = THREADS / kWave;
  const int NCH = W * SLABS;
  const int CPL = (NCH + kWave - 1) / kWave;
  static_assert(NCH % CPL == 0, "chunk table does not tile the lanes");
  static_assert(SLABS <= 32, "the per-wave masks have 32 bits");
  static_assert(kWave * N <= 256, "a list's length must fit the bits it is filed in");
  const int wave = __builtin_amdgcn_readfirstlane(WaveId());
  const int lane = LaneId();

  /* A: approximate sum and largest term of every chunk */
  MSHADOW_ROWSUM_STAMP(0)
  if (threadIdx.x == 0) {
    lds->s = 0.0f;
    lds->fail = 0;
    lds->nslots = 0u;
  }
  if (CHECK_SIGN) __syncthreads();  // the sign check below may set `fail`
  /* the wave-wide reductions take the slabs in groups of at most sixteen (registers) */
  const int GRP = SLABS < 16 ? SLABS : 16;
#pragma unroll
  for (int g = 0; g < SLABS; g += GRP) {
    float part[GRP];
#pragma unroll
    for (int j = 0; j < GRP; ++j) {
      part[j] = v[g + j][0];
#pragma unroll
      for (int i = 1; i < N; ++i) part[j] += v[g + j][i];
    }
    const float mine = mshadow::hip::WaveSumMany<GRP>(part);  // lane l: slab g + l % GRP
    if (lane < GRP) lds->approx[(g + lane) * W + wave] = mine;
    if (!UNIT_PEAK) {
      asm volatile("" ::: "memory");  // the two tables one after the other: fewer registers live
#pragma unroll
      for (int j = 0; j < GRP; ++j) {
        if (N == 4) {
          part[j] = MaxNum(MaxNum3(v[g + j][0], v[g + j][1 % N], v[g + j][2 % N]), v[g + j][3 % N]);
        } else {
          part[j] = v[g + j][0];
#pragma unroll
          for (int i = 1; i < N; ++i) part[j] = MaxNum(part[j], v[g + j][i]);
        }
      }
      const float most = mshadow::hip::WaveReduceMany<mshadow::hip::WaveOpMax, float, GRP>(part);
      if (lane < GRP) lds->cmax[(g + lane) * W + wave] = most;
    } else {
      /* The terms of a softmax are at most 1 and one of them is 1. A chunk's largest term
         serves as a lower bound of the sum behind it, and only a term next to a power of
         two - the 1 - tells more than the approximate sums do: the largest term is looked
         for only in chunks whose sum reaches 1, and taken as 0 elsewhere. */
      if (lane < GRP) lds->cmax[(g + lane) * W + wave] = 0.0f;
      for (uint32_t todo = static_cast<uint32_t>(__ballot(lane < GRP && mine >= 1.0f)); todo != 0u;
           todo &= todo - 1u) {
        const int j = g + __ffs(static_cast<int>(todo)) - 1;
        float t[N];
        SelectSlab<SLABS, N>(t, v, j);
        float m = t[0];
#pragma unroll
        for (int i = 1; i < N; ++i) m = MaxNum(m, t[i]);
        m = ReadLaneF32(mshadow::hip::WaveInclusiveScanMaxF32(m), kWave - 1);
        if (lane == 0) lds->cmax[j * W + wave] = m;
      }
    }
  }
  if (CHECK_SIGN) {  // the plan is made for non-negative terms
    float least = 0.0f;
#pragma unroll
    for (int j = 0; j < SLABS; ++j) {
#pragma unroll
      for (int i = 0; i < N; ++i) least = (v[j][i] < least) ? v[j][i] : least;
    }
    if (__ballot(least < 0.0f) != 0ull && lane == 0) lds->fail = 1;
  }
  __syncthreads();
  MSHADOW_ROWSUM_STAMP(1)

  /* B: plan per chunk, identical in every wave */
  uint32_t code[CPL];     // 1 + binade of a certain chunk, 0: to be listed
  uint32_t planned;       // how many chunks the plan lists
  {
    float pre[CPL + 1], seen[CPL + 1], own[CPL];
    pre[0] = 0.0f;
    seen[0] = 0.0f;
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const int k = lane * CPL + c;
      pre[c + 1] = pre[c] + (k < NCH ? lds->approx[k] : 0.0f);
      own[c] = k < NCH ? lds->cmax[k] : 0.0f;
      seen[c + 1] = MaxNum(seen[c], own[c]);
    }
    float incl = pre[CPL], seen_incl = seen[CPL];
    mshadow::hip::WaveScanSumAndMaxF32(&incl, &seen_incl);
    const float excl = incl - pre[CPL];
    const float approx_total = ReadLaneF32(incl, kWave - 1);
    /* a NaN among the terms makes the sum NaN whatever the order */
    if (approx_total != approx_total || s0 != s0) return s0 + approx_total;
    const float seen_excl = __uint_as_float(FromLaneBelowU32(__float_as_uint(seen_incl), 0u));
    /* the sum is never below a term already added */
    int raw[CPL];
    float st[CPL], lo[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const int k = lane * CPL + c;
      st[c] = s0 + (excl + pre[c]);
      /* s0, the sum in front of these terms, is itself a sum the row has reached */
      lo[c] = MaxNum(MaxNum3(PlanLowBound(st[c], static_cast<float>(k) * static_cast<float>(kWave * N)),
                             seen_excl, seen[c]), s0);
      raw[c] = PlanBinade(lo[c], PlanHighBound(s0 + (excl + pre[c + 1])));
    }
    /* neighbouring certain chunks must agree on the binade, or the later one is listed:
       every run of certain chunks then has one scale */
    const int before = static_cast<int>(FromLaneBelowU32(static_cast<uint32_t>(raw[CPL - 1]),
                                                         static_cast<uint32_t>(-1)));
    /* the chunks to be listed get their slots in row order, known to every wave alike; a
       chunk that turns out to hold a tie asks for one of the slots behind those */
    uint32_t in_lane[CPL];
    uint32_t mine = 0u, below = 0u;
    planned = 0u;
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const int prev = (c == 0) ? before : raw[c - 1];
      const bool clash = raw[c] >= 0 && prev >= 0 && prev != raw[c];
      code[c] = (raw[c] < 0 || clash) ? 0u : static_cast<uint32_t>(raw[c]) + 1u;
      const bool to_list = code[c] == 0u && lane * CPL + c < NCH;
      const unsigned long long listing = __ballot(to_list);
      in_lane[c] = mine;  // listed chunks of this lane in front of chunk c
      mine += to_list ? 1u : 0u;
      below += mshadow::hip::LanesBelow(listing);
      planned += static_cast<uint32_t>(__popcll(listing));
    }
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      typename Lds::ChunkPlan cp;
      cp.start = st[c];
      cp.low = lo[c];
      cp.slot = below + in_lane[c];
      cp.peak = own[c] > lo[c] ? 1u : 0u;
      if (lane * CPL + c < NCH) lds->plan[lane * CPL + c] = cp;
    }
  }

  /* C: integer totals of this wave's certain chunks ... */
  MSHADOW_ROWSUM_STAMP(2)
  uint32_t listed = 0u;  // this wave's slabs that go to the chain as lists
  static_assert(W % CPL == 0, "a wave's chunks must sit in one column of the chunk table");
  /* chunk j * W + wave sits in lane (j * W + wave) / CPL of table column wave % CPL */
  uint32_t my_code = code[0];
#pragma unroll
  for (int c = 1; c < CPL; ++c) my_code = (wave % CPL == c) ? code[c] : my_code;
  {
    /* Every certain chunk is quantised against its binade by two accumulators one ulp apart
       (LaneDualQuant); they end one ulp apart unless a term was a tie. The differences of
       all slabs are and-ed together: 1 exactly if every one of them is 1 (a lane that left
       its binade has a total that fails its run anyway). Only a wave that saw a tie looks
       for the slab it was in. */
    uint32_t all_gaps = 1u;
#pragma unroll
    for (int g = 0; g < SLABS; g += GRP) {
      uint32_t part[GRP];
#pragma unroll
      for (int j = 0; j < GRP; ++j) {
        const uint32_t ck = ReadLaneU32(my_code, ((g + j) * W + wave) / CPL);
        /* straight-line: a chunk to be listed is quantised too (against any binade) and
           its result dropped */
        const bool certain = ck != 0u;
        const uint32_t base = (certain ? ck - 1u : 1u) << 23;
        float lo = __uint_as_float(base), hi = __uint_as_float(base + 1u);
#pragma unroll
        for (int i = 0; i < N; ++i) {
          lo = lo + v[g + j][i];
          hi = hi + v[g + j][i];
        }
        all_gaps &= certain ? __float_as_uint(hi) - __float_as_uint(lo) : 1u;
        part[j] = __float_as_uint(lo) - base;
        listed |= certain ? 0u : 1u << (g + j);
      }
      const uint32_t total = mshadow::hip::WaveReduceMany<mshadow::hip::WaveOpSum, uint32_t, GRP>(part);
      /* lanes 0 .. GRP-1 file the result of "their" chunk (overwritten below if the chunk is
         listed after all); a total that cannot fit a binade is cut so that sums of totals
         stay inside 32 bits (the run it joins fails its check) */
      if (lane < GRP) lds->q[(g + lane) * W + wave] = total < (1u << 24) ? total : (1u << 24);
    }
    if (__ballot(all_gaps != 1u) != 0ull) {
      for (int j = 0; j < SLABS; ++j) {
        const uint32_t ck = ReadLaneU32(my_code, (j * W + wave) / CPL);
        if (ck == 0u) continue;
        float t[N];
        SelectSlab<SLABS, N>(t, v, j);
        if (__ballot(!LaneDualQuant<N>(t, ck - 1u).ok) != 0ull) listed |= 1u << j;
      }
    }
  }
  MSHADOW_ROWSUM_STAMP(6)
  /* ... and a list of addends for each of the others */
  for (uint32_t todo = listed; todo != 0u; todo &= todo - 1u) {
    const int j = __ffs(static_cast<int>(todo)) - 1;
    const int k = j * W + wave;
    const typename Lds::ChunkPlan cp = lds->plan[k];
    uint32_t slot;
    if (ReadLaneU32(my_code, k / CPL) == 0u) {
      slot = __builtin_amdgcn_readfirstlane(cp.slot);
    } else {
      slot = 0u;
      if (lane == 0) slot = planned + atomicAdd(&lds->nslots, 1u);
      slot = __builtin_amdgcn_readfirstlane(slot);
    }
    if (slot >= static_cast<uint32_t>(Lds::kSlots)) {  // no room: the row is redone by wave scans
      if (lane == 0) lds->fail = 1;
      break;
    }
    float t[N];
    SelectSlab<SLABS, N>(t, v, j);
    const float st = cp.start;
    const float lb = cp.low;
    /* the lane's own bounds: approximate prefix sums inside the chunk, and the largest term
       in front of it where that can raise the bound at all */
    float a = t[0];
#pragma unroll
    for (int i = 1; i < N; ++i) a += t[i];
    const float incl = WaveInclusiveScanF32(a);
    float lo = PlanLowBound(st + (incl - a), static_cast<float>(k * kWave + lane) * static_cast<float>(N));
    if (__builtin_amdgcn_readfirstlane(cp.peak) != 0u) {
      float m = t[0];
#pragma unroll
      for (int i = 1; i < N; ++i) m = MaxNum(m, t[i]);
      const float seen_incl = mshadow::hip::WaveInclusiveScanMaxF32(m);
      lo = MaxNum(lo, __uint_as_float(FromLaneBelowU32(__float_as_uint(seen_incl), 0u)));
    }
    lo = MaxNum(lo, lb);
    int c = PlanBinade(lo, PlanHighBound(st + incl));
    const LaneQuantum lq = LaneDualQuant<N>(t, c >= 0 ? static_cast<uint32_t>(c) : 1u);
    if (!lq.ok) c = -1;
    /* runs: maximal stretches of certain lanes with one binade; the first lane of a run
       files the run's addend, any other lane of it files nothing */
    const int below = static_cast<int>(FromLaneBelowU32(static_cast<uint32_t>(c), static_cast<uint32_t>(-1)));
    const bool term_lane = c < 0;
    const bool head = c >= 0 && below != c;
    const uint32_t qi = term_lane ? 0u : lq.q;
    const uint32_t q_incl = WaveInclusiveScanU32(qi);
    const unsigned long long terms = __ballot(term_lane);
    const unsigned long long heads = __ballot(head);
    const unsigned long long above = ((terms | heads) >> lane) >> 1;
    const int next_edge = above != 0ull ? lane + __ffsll(static_cast<long long>(above)) : kWave;
    const uint32_t q_end = static_cast<uint32_t>(__shfl(static_cast<int>(q_incl), next_edge - 1));
    /* place in the list: N per term lane and one per run in front of this lane */
    const uint32_t terms_below = __builtin_amdgcn_mbcnt_hi(
        static_cast<uint32_t>(terms >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(terms), 0u));
    const uint32_t heads_below = __builtin_amdgcn_mbcnt_hi(
        static_cast<uint32_t>(heads >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(heads), 0u));
    const uint32_t at = terms_below * N + heads_below;
    const uint32_t count = static_cast<uint32_t>(__popcll(terms)) * N + static_cast<uint32_t>(__popcll(heads));
    AddendList<N> *out = &lds->list[slot];
    if (term_lane) {
#pragma unroll
      for (int i = 0; i < N; ++i) {
        Addend e;
        e.value = t[i];
        e.check = 0u;
        out->entry[at + i] = e;
      }
    } else if (head) {
      Addend e;
      e.value = RunAddend(static_cast<uint32_t>(c), q_end - (q_incl - qi));
      e.check = static_cast<uint32_t>(c + 1);
      out->entry[at] = e;
    }
    if (lane == 0) lds->q[k] = kListedBit | (count << 8) | slot;
  }
  MSHADOW_ROWSUM_STAMP(8)
  __syncthreads();
  MSHADOW_ROWSUM_STAMP(3)

  /* D: the row's list of addends. Lane-parallel and the same in every wave: the listed
     chunks in row order, for each the addend of the run of certain chunks in front of it
     (their integer totals since the previous listed chunk, which share one binade) and the
     place of its list in the row's list; wave r % W then copies the list of listed chunk r. */
  if (lds->fail == 0) {
    uint32_t qk[CPL], pre[CPL + 1], cnt[CPL + 1], len[CPL + 1];
    pre[0] = 0u;
    cnt[0] = 0u;
    len[0] = 0u;
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      qk[c] = lane * CPL + c < NCH ? lds->q[lane * CPL + c] : 0u;
      const bool is_listed = (qk[c] & kListedBit) != 0u;
      if (is_listed) code[c] = 0u;  // planned certain, found to hold a tie
      pre[c + 1] = pre[c] + (is_listed ? 0u : qk[c]);
      cnt[c + 1] = cnt[c] + (is_listed ? 1u : 0u);
      len[c + 1] = len[c] + (is_listed ? ((qk[c] >> 8) & 0x1ffu) + 1u : 0u);
    }
    uint32_t incl = pre[CPL], cincl = cnt[CPL], lincl = len[CPL];
    mshadow::hip::WaveScanSum3U32(&incl, &cincl, &lincl);
    /* ex = integer total of the certain chunks in front of a chunk; it never decreases,
       so its value at the previous listed chunk is a running maximum */
    uint32_t own_last = 0u;
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      if ((qk[c] & kListedBit) != 0u) own_last = incl - pre[CPL] + pre[c];
    }
    const uint32_t last_incl = mshadow::hip::WaveInclusiveScanMaxU32(own_last);
    const uint32_t total_ex = ReadLaneU32(incl, kWave - 1);
    const uint32_t total_len = ReadLaneU32(lincl, kWave - 1) + 1u;  // + the run at the end
    const uint32_t last_ex = ReadLaneU32(last_incl, kWave - 1);
    uint32_t prev_ex = FromLaneBelowU32(last_incl, 0u);
    const uint32_t code_below = FromLaneBelowU32(code[CPL - 1], 0u);
    if (total_len > static_cast<uint32_t>(Lds::kRowAddends)) {
      if (threadIdx.x == 0) lds->fail = 1;
    } else {
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        const bool is_listed = (qk[c] & kListedBit) != 0u;
        const uint32_t ex = incl - pre[CPL] + pre[c];
        const uint32_t run = (c == 0) ? code_below : code[c - 1];
        const uint32_t rank = cincl - cnt[CPL] + cnt[c];
        const uint32_t at = lincl - len[CPL] + len[c];
        const float front = run != 0u ? RunAddend(run != 0u ? run - 1u : 0u, ex - prev_ex) : 0.0f;
        if (is_listed) prev_ex = ex;
        for (unsigned long long todo = __ballot(is_listed && rank % W == static_cast<uint32_t>(wave));
             todo != 0ull; todo &= todo - 1ull) {
          const int l = __ffsll(static_cast<long long>(todo)) - 1;
          const uint32_t q = ReadLaneU32(qk[c], l);
          const uint32_t to = ReadLaneU32(at, l);
          const float a0 = ReadLaneF32(front, l);
          const uint32_t c0 = ReadLaneU32(run, l);
          const AddendList<N> *from = &lds->list[q & 0xffu];
          const int n = static_cast<int>((q >> 8) & 0x1ffu);
          for (int g = lane; g < n; g += kWave) lds->row[to + 1u + g] = from->entry[g];
          if (lane == 0) {
            Addend e;
            e.value = a0;
            e.check = c0;
            lds->row[to] = e;
          }
        }
      }
      if (threadIdx.x == 0) {  // the run of certain chunks behind the last listed one
        const uint32_t run = TableAt<CPL>(code, NCH - 1);
        Addend e;
        e.value = run != 0u ? RunAddend(run - 1u, total_ex - last_ex) : 0.0f;
        e.check = run;
        lds->row[total_len - 1u] = e;
        lds->row_count = total_len;
      }
    }
  }
  __syncthreads();
  MSHADOW_ROWSUM_STAMP(4)

  /* E: the chain, in one wave */
  if (wave == 0 && lds->fail == 0) {
    /* the whole row waits for this chain; the other waves on this SIMD (another row's bulk
       phases) yield issue slots to it */
    __builtin_amdgcn_s_setprio(3);
    const int count = static_cast<int>(lds->row_count);
    float s = s0;
    bool bad = false;
    /* the next block is fetched while the current one is summed */
    Addend next;
    next.value = 0.0f;
    next.check = 0u;
    if (lane < count) next = lds->row[lane];
    for (int g0 = 0; g0 < count; g0 += kWave) {
      const Addend now = next;
      next.value = 0.0f;
      next.check = 0u;
      if (g0 + kWave + lane < count) next = lds->row[g0 + kWave + lane];
      const int left = count - g0;
      s = ChainBlock(s, now.value, now.check, left < kWave ? left : kWave, &bad);
    }
    const bool failed = __ballot(bad) != 0ull;
    if (lane == 0) {
      lds->s = s;
      if (failed) lds->fail = 1;
    }
    __builtin_amdgcn_s_setprio(0);
  }
  __syncthreads();
  MSHADOW_ROWSUM_STAMP(5)
  if (lds->fail == 0) return lds->s;
  MSHADOW_ROWSUM_STAMP(7)

  /* the plan did not hold (kept so that the result cannot depend on the plan): every chunk
     is resolved in row order by wave scans, wave after wave */
  __syncthreads();
  if (threadIdx.x == 0) lds->s = s0;
  __syncthreads();
  for (int j = 0; j < SLABS; ++j) {
    float t[N];
    SelectSlab<SLABS, N>(t, v, j);
    for (int w = 0; w < W; ++w) {
      if (wave == w) {
        const float r = WaveResolve<N>(lds->s, t);
        if (lane == 0) lds->s = r;
      }
      __syncthreads();
    }
  }
  return lds->s;
}

/*! \brief e^x for x <= 0 (any float accepted; -inf gives 0, NaN gives NaN), straight-line:
 *  h = 2^(x * log2(e) / 2) from the hardware exp2, with the rounding error of the product
 *  carried separately, then e^x = h * h * 2^r. The hardware exp2 does not return subnormals;
 *  h is a normal number whenever e^x is not zero, and the product h * h rounds correctly into
 *  the subnormal range. The result stays within about 3 ulp for the whole range a softmax
 *  sees. */
__device__ __forceinline__ float ExpNonPositive(float x) {
  const float kHalfLog2eHi = 0.5f * 1.44269502162933349609375f;
  const float kHalfLog2eLo = 0.5f * 1.925963033500011079013347625732421875e-08f;
  const float t = x * kHalfLog2eHi;
  float r = __builtin_fmaf(x, kHalfLog2eHi, -t);   // exact rounding error of the product
  r = __builtin_fmaf(x, kHalfLog2eLo, r);
  const float h = __builtin_amdgcn_exp2f(t);
  /* 2^(2 r) - 1 = r * 2 ln 2, |r| << 1. For x = -inf the error term is inf - inf: the NaN
     is dropped here (h is 0 then), while a NaN x still arrives through h. */
  const float c = MaxNum(r * 1.38629436111989061883f, -1.0f);
  const float e = h * h;
  return __builtin_fmaf(e, c, e);
}

/*! \brief p / s given rcp = 1 / s correctly rounded (s finite, at least 1): one multiply,
 *  within one ulp of the true quotient (half an ulp from the reciprocal, half from the
 *  product) */
__device__ __forceinline__ float DivideBy(float p, float /*s*/, float rcp) { return p * rcp; }

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

/*! \brief THREADS * SLABS * VEC >= cols. VEC == 4 moves 16-byte packs wherever the rows
 *  start and whatever their length (the last, partial pack of a row element by element). Slab j of wave w holds the 64 * VEC columns from (j * W + w) * 64 * VEC,
 *  lane l of that VEC consecutive ones: each load is one contiguous kilobyte per wave, the
 *  W waves together stream one contiguous stretch per slab, and the order of the row is
 *  slab, wave, lane, element.
 *  TERMS_GIVEN: src already holds the (non-negative) terms and dst[row] receives their
 *  left-to-right sum - the row-sum stage on its own. */
template <int THREADS, int SLABS, int VEC, bool TERMS_GIVEN, int MIN_WAVES = 4>
__global__ void __launch_bounds__(THREADS, MIN_WAVES)  // 4 waves per SIMD: two 512-thread rows per CU
    SoftmaxRowKernel(float *dst, int dstride, const float *src, int sstride, int cols) {
  __shared__ RowSumLds<THREADS / kWave, SLABS, VEC> lds;
  const int W = THREADS / kWave;
  const int kChunk = kWave * VEC;  // columns of one chunk
  const int wave = __builtin_amdgcn_readfirstlane(WaveId());
  const uint32_t lane_col = LaneId() * VEC;
  const float *in = src + static_cast<size_t>(blockIdx.x) * sstride;
  float *out = dst + static_cast<size_t>(blockIdx.x) * dstride;
  const float kNegInf = -__builtin_huge_valf();
  /* columns past the end of the row: -inf logits (their terms are exactly 0), zero terms */
  const float kAbsent = TERMS_GIVEN ? 0.0f : kNegInf;

  MSHADOW_ROWSUM_STAMP(10)
  /* chunk k = j * W + wave starts at column k * kChunk; whether it lies wholly inside the
     row is the same for all lanes, so the common case carries no per-lane guards */
  float v[SLABS][VEC];
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int c0 = (j * W + wave) * kChunk;
    const float *at = in + c0;  // uniform
    if (c0 + kChunk <= cols) {
      if (VEC == 4) {
        const F4 q = StreamLoadF4Anywhere(at + lane_col);
        v[j][0] = q.x; v[j][1 % VEC] = q.y; v[j][2 % VEC] = q.z; v[j][3 % VEC] = q.w;
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[j][i] = at[lane_col + i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[j][i] = kAbsent;
      if (VEC == 4) {  // whole packs as packs, the one the row ends in element by element
        if (c0 + static_cast<int>(lane_col) + VEC <= cols) {
          const F4 q = StreamLoadF4Anywhere(at + lane_col);
          v[j][0] = q.x; v[j][1 % VEC] = q.y; v[j][2 % VEC] = q.z; v[j][3 % VEC] = q.w;
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            if (c0 + static_cast<int>(lane_col) + i < cols) v[j][i] = at[lane_col + i];
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          if (c0 + static_cast<int>(lane_col) + i < cols) v[j][i] = at[lane_col + i];
        }
      }
    }
  }
  if (!TERMS_GIVEN) {
    float mx = kNegInf;
#pragma unroll
    for (int j = 0; j < SLABS; ++j) {
      if (VEC == 4) {
        mx = MaxNum3(mx, v[j][0], v[j][1 % VEC]);
        mx = MaxNum3(mx, v[j][2 % VEC], v[j][3 % VEC]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) mx = MaxNum(mx, v[j][i]);
      }
    }
    MSHADOW_ROWSUM_STAMP(11)
    mx = BlockMax<THREADS>(mx, lds.wmax);
    MSHADOW_ROWSUM_STAMP(12)
#pragma unroll
    for (int j = 0; j < SLABS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[j][i] = ExpNonPositive(v[j][i] - mx);
      /* one slab at a time: scheduled freely, the sixty-four independent chains would all
         be in flight at once and spill. The empty statement consumes this slab's results
         and hands out the next slab's inputs, so neither side can move across it. */
      if (j + 1 < SLABS) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) asm volatile("" : "+v"(v[j + 1][i]) : "v"(v[j][i]));
      }
    }
    MSHADOW_ROWSUM_STAMP(13)
  }

  const float s = RowOrderedSum<THREADS, SLABS, VEC, TERMS_GIVEN, !TERMS_GIVEN>(v, cols, &lds);
  if (TERMS_GIVEN) {
    if (threadIdx.x == 0) dst[blockIdx.x] = s;
    return;
  }

  /* s >= 1 for finite logits (the maximum contributes exp(0)); anything else (NaN or
     infinite logits) takes the plain division so that specials propagate as on the CPU */
  const bool fast_div = s >= 1.0f && s < 3.0e38f;
  const float rcp = 1.0f / s;
  if (!fast_div) {
#pragma unroll
    for (int j = 0; j < SLABS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[j][i] = v[j][i] / s;
    }
  }
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int c0 = (j * W + wave) * kChunk;
    float *at = out + c0;
    float o[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) o[i] = fast_div ? DivideBy(v[j][i], s, rcp) : v[j][i];
    if (VEC == 4) {
      F4 q;
      q.x = o[0]; q.y = o[1 % VEC]; q.z = o[2 % VEC]; q.w = o[3 % VEC];
      if (c0 + kChunk <= cols || c0 + static_cast<int>(lane_col) + VEC <= cols) {
        StreamStoreF4Anywhere(at + lane_col, q);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          if (c0 + static_cast<int>(lane_col) + i < cols) at[lane_col + i] = o[i];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        if (c0 + static_cast<int>(lane_col) + i < cols) at[lane_col + i] = o[i];
      }
    }
  }
  MSHADOW_ROWSUM_STAMP(14)
}

/*! \brief SLABS packs per thread of the stretch of a row that begins at `in` and has `left`
 *  columns to the end of the row, in the layout of SoftmaxRowKernel (slab j of wave w holds
 *  the 256 columns from (j * W + w) * 256): 16-byte accesses wherever the stretch starts, the
 *  pack the row ends in element by element, `absent` behind the end */
template <int THREADS, int SLABS>
__device__ __forceinline__ void LoadStretch(float (&v)[SLABS][4], const float *in, int left, float absent) {
  const int W = THREADS / kWave;
  const int wave = __builtin_amdgcn_readfirstlane(WaveId());
  const int lane_col = LaneId() * 4;
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int c0 = (j * W + wave) * 256;  // uniform
    const float *at = in + c0 + lane_col;
    if (c0 + 256 <= left || c0 + lane_col + 4 <= left) {
      const F4 q = StreamLoadF4Anywhere(at);
      v[j][0] = q.x; v[j][1] = q.y; v[j][2] = q.z; v[j][3] = q.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[j][i] = (c0 + lane_col + i < left) ? at[i] : absent;
    }
  }
}

/*! \brief rows longer than one workgroup's registers hold (more than THREADS * SLABS * 4
 *  columns), any length: one workgroup per row takes the row stretch by stretch, three times -
 *  the maximum; the terms exp(x - max) of each stretch and their sum, which RowOrderedSum
 *  continues from the sum of the stretches in front (so the row's sum is the left-to-right sum
 *  of mshadow/tensor_cpu-inl.h:277-281 as in the kernel above); the terms once more (the same
 *  instructions on the same logits give the same terms), divided and stored. src is read three
 *  times, the second and third time mostly from the caches, dst written once; dst may alias src
 *  (a thread reads a pack for the last time before it writes it).
 *  TERMS_GIVEN: src already holds the (non-negative) terms and dst[row] receives their
 *  left-to-right sum - the row-sum stage on its own, one pass.
 *  MIN_WAVES (per SIMD): 4 fits two 512-thread rows on a CU at the price of a few registers kept
 *  in scratch memory - faster when there are more rows than CUs ((512,128000): 204 against
 *  224 us), slower when there are not ((16,250000): 129 against 113 us), where 2 is used. */
template <int THREADS, int SLABS, bool TERMS_GIVEN, int MIN_WAVES>
__global__ void __launch_bounds__(THREADS, MIN_WAVES)
    SoftmaxStretchRowKernel(float *dst, int dstride, const float *src, int sstride, int cols) {
  __shared__ RowSumLds<THREADS / kWave, SLABS, 4> lds;
  const int W = THREADS / kWave;
  const int kStretch = THREADS * SLABS * 4;
  const int wave = __builtin_amdgcn_readfirstlane(WaveId());
  const int lane_col = LaneId() * 4;
  const float *in = src + static_cast<size_t>(blockIdx.x) * sstride;
  float *out = dst + static_cast<size_t>(blockIdx.x) * dstride;
  const float kNegInf = -__builtin_huge_valf();
  float v[SLABS][4];
  float mx = kNegInf;
  if (!TERMS_GIVEN) {
    for (int t0 = 0; t0 < cols; t0 += kStretch) {
      LoadStretch<THREADS, SLABS>(v, in + t0, cols - t0, kNegInf);
#pragma unroll
      for (int j = 0; j < SLABS; ++j) {
        mx = MaxNum3(mx, v[j][0], v[j][1]);
        mx = MaxNum3(mx, v[j][2], v[j][3]);
      }
    }
    mx = BlockMax<THREADS>(mx, lds.wmax);
  }
  float s = 0.0f;
  for (int t0 = 0; t0 < cols; t0 += kStretch) {
    LoadStretch<THREADS, SLABS>(v, in + t0, cols - t0, TERMS_GIVEN ? 0.0f : kNegInf);
    if (!TERMS_GIVEN) {
#pragma unroll
      for (int j = 0; j < SLABS; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[j][i] = ExpNonPositive(v[j][i] - mx);
        if (j + 1 < SLABS) {  // one slab at a time, as in SoftmaxRowKernel
#pragma unroll
          for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(v[j + 1][i]) : "v"(v[j][i]));
        }
      }
    }
    __syncthreads();  // everybody has read the sum the stretch in front left in LDS
    s = RowOrderedSum<THREADS, SLABS, 4, TERMS_GIVEN, !TERMS_GIVEN>(v, cols - t0, &lds, s);
  }
  if (TERMS_GIVEN) {
    if (threadIdx.x == 0) dst[blockIdx.x] = s;
    return;
  }
  const bool fast_div = s >= 1.0f && s < 3.0e38f;
  const float rcp = 1.0f / s;
  for (int t0 = 0; t0 < cols; t0 += kStretch) {
    const int left = cols - t0;
    LoadStretch<THREADS, SLABS>(v, in + t0, left, kNegInf);
#pragma unroll
    for (int j = 0; j < SLABS; ++j) {
      const int c0 = (j * W + wave) * 256;
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = ExpNonPositive(v[j][i] - mx);
        o[i] = fast_div ? DivideBy(p, s, rcp) : p / s;
      }
      float *at = out + t0 + c0 + lane_col;
      if (c0 + 256 <= left || c0 + lane_col + 4 <= left) {
        F4 q;
        q.x = o[0]; q.y = o[1]; q.z = o[2]; q.w = o[3];
        StreamStoreF4Anywhere(at, q);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (c0 + lane_col + i < left) at[i] = o[i];
        }
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

/*! \brief WaveResolve for four or two rows side by side in one wave, one to each group of LANES =
 *  16 (a DPP row) or 32 lanes: every group adds its LANES * N terms (lane order, then element
 *  order) to its own s exactly as a serial loop would. The scans stop at the groups' borders; a
 *  group that is done idles while the others finish. Every lane of the wave must call it. */
template <int LANES, int N>
__device__ inline float PartWaveResolve(float s, const float (&t)[N]) {
  using namespace ordered_sum;
  static_assert(LANES == 16 || LANES == 32, "a quarter or a half of a wave");
  const int lane = LaneId();
  const int l = lane & (LANES - 1), first_lane = lane & ~(LANES - 1);
  int start = 0;
  bool done = false;
  while (true) {
    const Binade b = BinadeOf(s);
    const bool active = !done && l >= start;
    float incl = active ? LaneQuant<N>(t, b) : 0.0f;
#define MSHADOW_ROWSCAN_STEP(SH) \
    incl += __uint_as_float(mshadow::hip::DppU32<MSHADOW_DPP_ROW_SHR(SH), 0xf>(0u, __float_as_uint(incl)));
    MSHADOW_ROWSCAN_STEP(1)
    MSHADOW_ROWSCAN_STEP(2)
    MSHADOW_ROWSCAN_STEP(4)
    MSHADOW_ROWSCAN_STEP(8)
#undef MSHADOW_ROWSCAN_STEP
    if (LANES == 32) {  // lane 15 of rows 0 and 2 to every lane of rows 1 and 3
      incl += __uint_as_float(mshadow::hip::DppU32<MSHADOW_DPP_ROW_BCAST15, 0xa>(0u, __float_as_uint(incl)));
    }
    const bool fail = active && !Fits(b, incl);
    const unsigned long long mask = __ballot(fail);
    const uint32_t mine = static_cast<uint32_t>(mask >> first_lane) & (LANES == 32 ? 0xffffffffu : 0xffffu);
    const int first = mine ? __ffs(static_cast<int>(mine)) - 1 : LANES;
    /* what the lanes in front of `first` add is exact (their inclusive prefix is) */
    const float upto = __shfl(incl, first_lane + (first > 0 ? first - 1 : 0));
    const float s1 = Accept(s, b, first > 0 ? upto : 0.0f);
    /* lane `first` does real float adds; every lane computes, one result is taken */
    const float s2 = __shfl(TrueAdd<N>(s1, t), first_lane + (first < LANES ? first : LANES - 1));
    if (!done) {
      s = first < LANES ? s2 : s1;
      start = first + 1;
      done = start >= LANES;
    }
    if (__all(done)) return s;
  }
}

/*! \brief four or two rows per wave, LANES = 16 or 32 lanes each, cols <= LANES * N: lane l of a
 *  row's group holds the N consecutive columns from l * N. The wave-wide steps of a row - the
 *  maximum, the scans of the ordered sum - cost the same instructions whether a wave holds one
 *  short row or four, and rows of up to 256 columns by the hundred thousand are bound by
 *  exactly those. 256 / LANES rows per workgroup, nothing shared between them, no barrier. */
template <int LANES, int N, bool TERMS_GIVEN>
__global__ void __launch_bounds__(256)
    SoftmaxPartWaveKernel(float *dst, int dstride, const float *src, int sstride, int rows, int cols) {
  const int row = blockIdx.x * (256 / LANES) + static_cast<int>(threadIdx.x) / LANES;
  const bool there = row < rows;
  const int rowc = there ? row : rows - 1;   // every lane takes part in the wave-wide steps
  const int lane = LaneId();
  const int base = (lane & (LANES - 1)) * N;
  const float *in = src + static_cast<size_t>(rowc) * sstride;
  const float kNegInf = -__builtin_huge_valf();
  const float kAbsent = TERMS_GIVEN ? 0.0f : kNegInf;
  float v[N];
#pragma unroll
  for (int p = 0; p < N; p += 4) {
    if (base + p + 4 <= cols) {
      const F4 q = StreamLoadF4Anywhere(in + base + p);
      v[p] = q.x; v[p + 1] = q.y; v[p + 2] = q.z; v[p + 3] = q.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[p + i] = (base + p + i < cols) ? in[base + p + i] : kAbsent;
    }
  }
  if (!TERMS_GIVEN) {
    float mx = kNegInf;
#pragma unroll
    for (int i = 0; i < N; ++i) mx = (mx < v[i]) ? v[i] : mx;
#define MSHADOW_ROWMAX_STEP(SH)                                                                   \
    {                                                                                             \
      const float o = __uint_as_float(mshadow::hip::DppU32<MSHADOW_DPP_ROW_SHR(SH), 0xf>(         \
          __float_as_uint(mx), __float_as_uint(mx)));                                             \
      mx = (mx < o) ? o : mx;                                                                     \
    }
    MSHADOW_ROWMAX_STEP(1)
    MSHADOW_ROWMAX_STEP(2)
    MSHADOW_ROWMAX_STEP(4)
    MSHADOW_ROWMAX_STEP(8)
#undef MSHADOW_ROWMAX_STEP
    if (LANES == 32) {
      const float o = __uint_as_float(mshadow::hip::DppU32<MSHADOW_DPP_ROW_BCAST15, 0xa>(
          __float_as_uint(mx), __float_as_uint(mx)));
      mx = (mx < o) ? o : mx;
    }
    mx = __shfl(mx, lane | (LANES - 1));   // the group's last lane holds the maximum of all its lanes
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = (base + i < cols) ? ExpNonPositive(v[i] - mx) : 0.0f;
  }
  const float s = PartWaveResolve<LANES, N>(0.0f, v);
  if (!there) return;
  if (TERMS_GIVEN) {
    if ((lane & (LANES - 1)) == 0) dst[row] = s;
    return;
  }
  float *out = dst + static_cast<size_t>(row) * dstride;
  const bool fast_div = s >= 1.0f && s < 3.0e38f;
  const float rcp = 1.0f / s;
#pragma unroll
  for (int p = 0; p < N; p += 4) {
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = fast_div ? DivideBy(v[p + i], s, rcp) : v[p + i] / s;
    if (base + p + 4 <= cols) {
      F4 q;
      q.x = o[0]; q.y = o[1]; q.z = o[2]; q.w = o[3];
      StreamStoreF4Anywhere(out + base + p, q);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (base + p + i < cols) out[base + p + i] = o[i];
      }
    }
  }
}

/*! \brief one wave per row, cols <= 256 * SLABS: slab k is the 256 columns from 256 * k, lane l
 *  holds the four from 256 * k + 4 * l (every load and store of the wave is one contiguous
 *  kilobyte), and the sum is resolved slab after slab, in lane order within a slab
 *  (WaveResolve) - the row's own order. Four rows per workgroup, nothing shared between them,
 *  no barrier: for rows of a few hundred to a few thousand columns, where a workgroup per row
 *  spends its time in the barriers of the long-row plan (65536 x 1000: 194 us). */
template <int SLABS, bool TERMS_GIVEN>
__global__ void __launch_bounds__(256)
    SoftmaxWaveSlabsKernel(float *dst, int dstride, const float *src, int sstride, int rows,
                           int cols) {
  const int row = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(WaveId());
  if (row >= rows) return;
  const int lane_col = LaneId() * 4;
  const float *in = src + static_cast<size_t>(row) * sstride;
  const float kNegInf = -__builtin_huge_valf();
  const float kAbsent = TERMS_GIVEN ? 0.0f : kNegInf;
  float v[SLABS][4];
  float mx = kNegInf;
#pragma unroll
  for (int k = 0; k < SLABS; ++k) {
    const int c = k * 256 + lane_col;
    if (c + 4 <= cols) {
      const F4 q = StreamLoadF4Anywhere(in + c);
      v[k][0] = q.x; v[k][1] = q.y; v[k][2] = q.z; v[k][3] = q.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[k][i] = (c + i < cols) ? in[c + i] : kAbsent;
    }
    mx = MaxNum3(mx, v[k][0], v[k][1]);
    mx = MaxNum3(mx, v[k][2], v[k][3]);
  }
  if (!TERMS_GIVEN) {
    mx = WaveMaxF32(mx);
#pragma unroll
    for (int k = 0; k < SLABS; ++k) {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[k][i] = ExpNonPositive(v[k][i] - mx);
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int k = 0; k < SLABS; ++k) {
    if (k * 256 < cols) s = WaveResolve<4>(s, v[k]);
  }
  if (TERMS_GIVEN) {
    if (LaneId() == 0) dst[row] = s;
    return;
  }
  float *out = dst + static_cast<size_t>(row) * dstride;
  const bool fast_div = s >= 1.0f && s < 3.0e38f;
  const float rcp = 1.0f / s;
#pragma unroll
  for (int k = 0; k < SLABS; ++k) {
    const int c = k * 256 + lane_col;
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = fast_div ? DivideBy(v[k][i], s, rcp) : v[k][i] / s;
    if (c + 4 <= cols) {
      F4 q;
      q.x = o[0]; q.y = o[1]; q.z = o[2]; q.w = o[3];
      StreamStoreF4Anywhere(out + c, q);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (c + i < cols) out[c + i] = o[i];
      }
    }
  }
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
      if (x + 4 <= cols) q[u] = StreamLoadF4Anywhere(in + x);
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
        StreamStoreF4Anywhere(out + x, q[u]);
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

/*! \brief the same for rows of up to 512 columns, where a workgroup per row leaves most of its
 *  threads idle: a workgroup takes kGradBlock / ppr consecutive rows, ppr = ceil(cols / 4) packs
 *  each (`div_ppr` divides by it), a thread one pack. grid.x = ceil(rows / rows_per_block). */
template <int FLAGS>
__global__ void __launch_bounds__(kGradBlock)
    SoftmaxGradShortRowsKernel(float *dst, int dstride, const float *src, int sstride, const float *label,
                               int rows, int cols, int rows_per_block, mshadow::FastDivU32 div_ppr,
                               GradParams gp) {
  const uint32_t r = div_ppr.Div(threadIdx.x);
  const int y = blockIdx.x * rows_per_block + static_cast<int>(r);
  if (static_cast<int>(r) >= rows_per_block || y >= rows) return;
  const int x = static_cast<int>(threadIdx.x - r * div_ppr.div) * 4;
  const int k = static_cast<int>(label[y]);
  const bool ignored = (FLAGS & kGradIgnore) && k == gp.ignore_label;
  const float *in = src + static_cast<size_t>(y) * sstride;
  float *out = dst + static_cast<size_t>(y) * dstride;
  if (x + 4 <= cols) {
    F4 q = StreamLoadF4Anywhere(in + x);
    q.x = GradElement<FLAGS>(q.x, k == x, ignored, gp);
    q.y = GradElement<FLAGS>(q.y, k == x + 1, ignored, gp);
    q.z = GradElement<FLAGS>(q.z, k == x + 2, ignored, gp);
    q.w = GradElement<FLAGS>(q.w, k == x + 3, ignored, gp);
    StreamStoreF4Anywhere(out + x, q);
  } else {
    for (int i = x; i < cols; ++i) out[i] = GradElement<FLAGS>(in[i], i == k, ignored, gp);
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
