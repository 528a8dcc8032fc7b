/*
 * Softmax / SoftmaxGrad for element types other than float (half_t, double), written in the
 * element type's own arithmetic so that every intermediate rounds where the CPU path rounds
 * (mshadow/tensor_cpu-inl.h:270-302): the difference x - max, the exponential stored into
 * dst, the running sum after every add and the final quotient are all values of DType.
 * For half_t that matters: a sum kept in 16 bits stops growing once its ulp exceeds twice the
 * terms (4096 equal logits give 1/2048 each, not 1/4096), and only the left-to-right order
 * reproduces it.
 *
 * A workgroup of 256 threads takes kAnyRows = 8 rows, 32 threads per row, each thread four
 * packs of kAnyTile = 8 consecutive elements per step (128-bit accesses for half_t when rows are
 * aligned whole packs; a row is visited in contiguous stretches of 1024 elements). The maximum
 * is a reduction over the row's 32 threads (exact in any order). The rows then pass in tiles
 * of 1024 columns: every thread computes its packs of terms (the next tile's logits are
 * already on their way), stores them to dst and parks them in LDS; eight lanes of one wave
 * then each add one row's 1024 terms to that row's running sum, term by term, four packs
 * being added while the next four come from LDS, and while the other waves make the next
 * tile in the second LDS buffer. A wave instruction costs the same for one active lane as
 * for sixty-four, so the chains of the eight rows share their instructions (one wave per
 * row: 1457 us for 8192 x 32000 half_t; this kernel: 670 us, of which the five passes over
 * memory - logits twice, terms written, read back and written again - would take about 440
 * at the rate of a plain copy; four or sixteen rows per workgroup were slower, as was making
 * the terms a second time from the logits instead of storing them and reading them back).
 * A last pass divides the stored terms. A thread only ever reads back and writes the
 * elements it handled itself, so in-place calls (dst == src) are safe.
 *
 * The float versions are the fixed-function kernels of the library (csrc/softmax_kernels.h).
 */
#ifndef MSHADOW_HIP_KERNELS_SOFTMAX_ANY_H_
#define MSHADOW_HIP_KERNELS_SOFTMAX_ANY_H_

#include "../../half.h"
#include "./common.h"
#include "./half_prune.h"

namespace mshadow {
namespace hip {

const int kAnyBlock = 256;
/*! \brief rows per workgroup */
const int kAnyRows = 8;
/*! \brief consecutive elements of one thread per step */
const int kAnyTile = 8;
const int kAnyThreadsPerRow = kAnyBlock / kAnyRows;
/*! \brief packs of one thread per step: a row is visited in stretches of
 *  kAnyBatch * kAnyThreadsPerRow packs (2 KB of half_t), pack q of thread p being pack
 *  q * kAnyThreadsPerRow + p of the stretch, so that a wave's accesses stay contiguous */
const int kAnyBatch = 4;
const int kAnyStepCols = kAnyThreadsPerRow * kAnyTile;
const int kAnyTileCols = kAnyBatch * kAnyStepCols;
/*! \brief row pitch of the LDS tile: one pack more than it holds, so that the eight chain
 *  lanes read from different banks */
const int kAnyPitch = kAnyTileCols + kAnyTile;

template <typename DType>
struct alignas(16) AnyPack {
  DType v[kAnyTile];
};

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

/*! \brief sum += t as DType does it. For half_t one 16-bit add: it rounds the exact sum once,
 *  which equals widening, adding in float and rounding back (24 >= 2 * 11 + 2 bits), and is a
 *  third of the dependent instructions. */
template <typename DType>
__device__ __forceinline__ void ChainAdd(DType &sum, const DType &t) { sum += t; }
__device__ __forceinline__ void ChainAdd(half::half_t &sum, const half::half_t &t) {
  const _Float16 a = __builtin_bit_cast(_Float16, sum.half_);
  const _Float16 b = __builtin_bit_cast(_Float16, t.half_);
  sum.half_ = __builtin_bit_cast(uint16_t, static_cast<_Float16>(a + b));
}

/*! \brief elements [x, x + kAnyTile) of a row; VEC: whole aligned packs only */
template <typename DType, bool VEC>
__device__ __forceinline__ void LoadAnyPack(AnyPack<DType> *p, const DType *row, uint32_t x,
                                            uint32_t cols, DType absent) {
  if (VEC) {
    *p = *reinterpret_cast<const AnyPack<DType> *>(row + x);
  } else {
#pragma unroll
    for (int i = 0; i < kAnyTile; ++i) p->v[i] = (x + i < cols) ? row[x + i] : absent;
  }
}
template <typename DType, bool VEC>
__device__ __forceinline__ void StoreAnyPack(DType *row, uint32_t x, uint32_t cols,
                                             const AnyPack<DType> &p) {
  if (VEC) {
    *reinterpret_cast<AnyPack<DType> *>(row + x) = p;
  } else {
#pragma unroll
    for (int i = 0; i < kAnyTile; ++i) {
      if (x + i < cols) row[x + i] = p.v[i];
    }
  }
}

/*! \brief VEC: cols % kAnyTile == 0 and every row of src and dst starts 16-byte aligned */
template <typename DType, bool VEC>
__global__ void __launch_bounds__(kAnyBlock)
    SoftmaxAnyKernel(DType *dst, uint32_t dstride, const DType *src, uint32_t sstride,
                     uint32_t rows, uint32_t cols) {
  typedef typename WideOf<DType>::Type Wide;
  __shared__ AnyPack<DType> tile_packs[2][kAnyRows][kAnyPitch / kAnyTile];
  __shared__ DType sums[kAnyRows];
  const uint32_t r = threadIdx.x / kAnyThreadsPerRow;
  const uint32_t p = threadIdx.x % kAnyThreadsPerRow;
  const uint32_t row = blockIdx.x * kAnyRows + r;
  /* threads without a row run along (the barriers are the workgroup's) and touch nothing */
  const bool live = row < rows;
  const DType *e = src + static_cast<size_t>(live ? row : 0) * sstride;
  DType *o = dst + static_cast<size_t>(live ? row : 0) * dstride;

  /* maximum: `if (mmax < e[x]) mmax = e[x]` from e[0] on, which is the largest value */
  const DType first = e[0];
  Wide m = static_cast<Wide>(first);
  if (live) {
    for (uint32_t x0 = 0; x0 < cols; x0 += kAnyTileCols) {
      AnyPack<DType> in[kAnyBatch];
#pragma unroll
      for (int q = 0; q < kAnyBatch; ++q) {
        const uint32_t x = x0 + (q * kAnyThreadsPerRow + p) * kAnyTile;
        if (x < cols) {
          LoadAnyPack<DType, VEC>(&in[q], e, x, cols, first);
        } else {
#pragma unroll
          for (int i = 0; i < kAnyTile; ++i) in[q].v[i] = first;
        }
      }
#pragma unroll
      for (int q = 0; q < kAnyBatch; ++q) {
#pragma unroll
        for (int i = 0; i < kAnyTile; ++i) {
          const Wide v = static_cast<Wide>(in[q].v[i]);
          m = (m < v) ? v : m;
        }
      }
    }
  }
#pragma unroll
  for (int d = 1; d < kAnyThreadsPerRow; d <<= 1) {  // the row's 32 threads are half a wave
    const Wide other = WaveShuffleXor(m, d);
    m = (m < other) ? other : m;
  }
  const DType mmax = static_cast<DType>(m);  // exact: m is one of the row's values

  /* chain lane c (lane c < kAnyRows of one wave) owns the running sum of row c. Which wave
     does it rotates with the workgroup number, so that the chains of the workgroups sharing
     a CU sit on different SIMDs */
  const uint32_t chain_wave = blockIdx.x % (kAnyBlock / kWave);
  const uint32_t c = threadIdx.x & (kWave - 1);
  const bool chain_slot = (threadIdx.x >> 6) == chain_wave && c < static_cast<uint32_t>(kAnyRows);
  const bool chain_lane = chain_slot && blockIdx.x * kAnyRows + c < rows;
  DType sum = DType(0.0f);
  /* the packs of the next tile are fetched before this tile's terms are computed and summed */
  AnyPack<DType> in[kAnyBatch];
#pragma unroll
  for (int q = 0; q < kAnyBatch; ++q) {
    const uint32_t x = (q * kAnyThreadsPerRow + p) * kAnyTile;
    if (live && x < cols) LoadAnyPack<DType, VEC>(&in[q], e, x, cols, mmax);
  }
  /* Tile i's terms are added while tile i + 1 is being made: in step i every thread makes its
     packs of tile i (LDS buffer i & 1), then the chain lanes add tile i - 1 from the other
     buffer, then all meet. One step more than there are tiles adds the last one. A buffer is
     written again two steps after it was written, one barrier after it was last read. */
  const uint32_t ntiles = (cols + kAnyTileCols - 1) / kAnyTileCols;
  for (uint32_t step = 0; step <= ntiles; ++step) {
    const uint32_t x0 = step * kAnyTileCols;
    if (step < ntiles) {
      AnyPack<DType> next[kAnyBatch];
#pragma unroll
      for (int q = 0; q < kAnyBatch; ++q) {
        const uint32_t x = x0 + kAnyTileCols + (q * kAnyThreadsPerRow + p) * kAnyTile;
        if (live && x < cols) LoadAnyPack<DType, VEC>(&next[q], e, x, cols, mmax);
      }
#pragma unroll
      for (int q = 0; q < kAnyBatch; ++q) {
        const uint32_t x = x0 + (q * kAnyThreadsPerRow + p) * kAnyTile;
        if (live && x < cols) {
          AnyPack<DType> t;
#pragma unroll
          for (int i = 0; i < kAnyTile; ++i) t.v[i] = DType(SoftmaxExp(in[q].v[i] - mmax));
          StoreAnyPack<DType, VEC>(o, x, cols, t);
          tile_packs[step & 1u][r][q * kAnyThreadsPerRow + p] = t;
        }
      }
#pragma unroll
      for (int q = 0; q < kAnyBatch; ++q) in[q] = next[q];
    }
    if (chain_lane && step > 0) {
      const uint32_t done = x0 - kAnyTileCols;  // first column of the tile being added
      const uint32_t n = cols - done < static_cast<uint32_t>(kAnyTileCols) ? cols - done : kAnyTileCols;
      const AnyPack<DType> *mine = tile_packs[(step - 1u) & 1u][c];
      const uint32_t full = n / kAnyTile;  // whole packs
      uint32_t k = 0;
      if (full >= 4) {
        /* four packs are added while the next four are on their way from LDS */
        AnyPack<DType> a[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) a[q] = mine[q];
        for (; k + 8 <= full; k += 4) {
          AnyPack<DType> b[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) b[q] = mine[k + 4 + q];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
#pragma unroll
            for (int i = 0; i < kAnyTile; ++i) ChainAdd(sum, a[q].v[i]);
          }
#pragma unroll
          for (int q = 0; q < 4; ++q) a[q] = b[q];
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
#pragma unroll
          for (int i = 0; i < kAnyTile; ++i) ChainAdd(sum, a[q].v[i]);
        }
        k += 4;
      }
      for (; k < full; ++k) {
        const AnyPack<DType> t = mine[k];
#pragma unroll
        for (int i = 0; i < kAnyTile; ++i) ChainAdd(sum, t.v[i]);
      }
      if (k * kAnyTile < n) {
        const AnyPack<DType> t = mine[k];
#pragma unroll
        for (int i = 0; i < kAnyTile; ++i) {  // unrolled: a run-time index would put t in scratch memory
          if (k * kAnyTile + i < n) ChainAdd(sum, t.v[i]);
        }
      }
    }
    __syncthreads();
  }
  if (chain_slot) sums[c] = sum;
  __syncthreads();
  sum = sums[r];

  /* every thread reads back only what it stored itself */
  if (live) {
    for (uint32_t x0 = 0; x0 < cols; x0 += kAnyTileCols) {
      AnyPack<DType> t[kAnyBatch];
#pragma unroll
      for (int q = 0; q < kAnyBatch; ++q) {
        const uint32_t x = x0 + (q * kAnyThreadsPerRow + p) * kAnyTile;
        if (x < cols) LoadAnyPack<DType, VEC>(&t[q], o, x, cols, sum);
      }
#pragma unroll
      for (int q = 0; q < kAnyBatch; ++q) {
        const uint32_t x = x0 + (q * kAnyThreadsPerRow + p) * kAnyTile;
        if (x < cols) {
#pragma unroll
          for (int i = 0; i < kAnyTile; ++i) t[q].v[i] /= sum;
          StoreAnyPack<DType, VEC>(o, x, cols, t[q]);
        }
      }
    }
  }
}

/* ---- long binary16 rows, kept on chip ---------------------------------------------------
 * A row of up to 32768 half_t is 64 KB: a 256-thread workgroup holds it in registers (sixteen
 * packs of eight per thread, pack q of thread t being columns (q * 256 + t) * 8 ..), so the
 * logits are read once and the probabilities written once - two passes over memory instead
 * of five. What remains is the row sum, 32000 dependent 16-bit adds in the reference's order
 * (mshadow/tensor_cpu-inl.h:277-281 with DType = half_t). Most of them change nothing
 * (half_prune.h): the row is walked in stretches of 2048 columns, the largest term of the
 * stretches already passed is a lower bound of the running sum, and only the terms that can
 * still change a sum that large are copied, in row order, to a list in LDS. One thread then
 * adds the list - a few thousand entries for a softmax over 32000 classes - term by term. A
 * row whose list would not fit (rows of equal logits: every term counts until the sum stops
 * at 2048) is summed stretch by stretch with all its terms instead. Either way the sum sees
 * exactly the adds that change it, in order: bit-identical to the serial loop. */
const int kHalfRowBlock = 256;
const int kHalfRowPacks = 16;
static_assert(kHalfRowPacks * (kHalfRowBlock / kWave) == kWave, "a lane per run of the row");
const int kHalfRowStretch = kHalfRowBlock * kAnyTile;
const int kHalfRowMaxCols = kHalfRowPacks * kHalfRowStretch;
/*! \brief rows shorter than this go several to a workgroup (SoftmaxAnyKernel) */
const int kHalfRowMinCols = 4096;
/*! \brief entries of the list of terms that count (32 KB of LDS: four rows resident per CU) */
const int kHalfRowList = 16384;

/*! \brief a pack of eight binary16 values as four 32-bit words: arrays of half_t in registers
 *  take a register per element, these a register per two */
typedef uint32_t HalfPackWords __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint32_t HalfBitsAt(const HalfPackWords &p, int i) {
  return (p[i >> 1] >> ((i & 1) * 16)) & 0xffffu;
}
__device__ __forceinline__ void SetHalfBitsAt(HalfPackWords &p, int i, uint32_t bits) {
  const uint32_t keep = (i & 1) ? 0x0000ffffu : 0xffff0000u;
  p[i >> 1] = (p[i >> 1] & keep) | (bits << ((i & 1) * 16));
}

/*! \brief sum += the eight values of a pack, in order, one 16-bit add each */
__device__ __forceinline__ void ChainAddPack(_Float16 &sum, const HalfPackWords &p) {
#pragma unroll
  for (int i = 0; i < kAnyTile; ++i) {
    sum = sum + __builtin_bit_cast(_Float16, static_cast<uint16_t>(HalfBitsAt(p, i)));
  }
}

/*! \brief sum += list[0 .. n) in order, one 16-bit add per entry; eight entries per LDS read,
 *  four reads in flight while the previous four are added (list is in LDS, 16-byte aligned) */
__device__ __forceinline__ uint32_t ChainHalfList(uint32_t sum_bits, const uint16_t *list, uint32_t n) {
  typedef __attribute__((address_space(3))) const HalfPackWords LdsPack;
  typedef __attribute__((address_space(3))) const uint16_t LdsHalf;
  _Float16 sum = __builtin_bit_cast(_Float16, static_cast<uint16_t>(sum_bits));
  LdsPack *packs = (LdsPack *)list;
  const uint32_t full = n / kAnyTile;
  uint32_t k = 0;
  if (full >= 4) {
    HalfPackWords a[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) a[q] = packs[q];
    for (; k + 8 <= full; k += 4) {
      HalfPackWords b[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) b[q] = packs[k + 4 + q];
#pragma unroll
      for (int q = 0; q < 4; ++q) ChainAddPack(sum, a[q]);
#pragma unroll
      for (int q = 0; q < 4; ++q) a[q] = b[q];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) ChainAddPack(sum, a[q]);
    k += 4;
  }
  for (; k < full; ++k) {
    const HalfPackWords one = packs[k];
    ChainAddPack(sum, one);
  }
  LdsHalf *tail = (LdsHalf *)list;
  for (uint32_t j = full * kAnyTile; j < n; ++j) sum = sum + __builtin_bit_cast(_Float16, tail[j]);
  return __builtin_bit_cast(uint16_t, sum);
}

/*! \brief work on `next` may not start before the work on `done` is finished: scheduled
 *  freely, the independent chains of all sixteen packs would be in flight at once and spill.
 *  The empty statement consumes one pack's results and hands out the other's inputs. */
__device__ __forceinline__ void OnePackAtATime(HalfPackWords &done, HalfPackWords &next) {
  /* `done` is an output too: what the compiler knows of how its words were put together (the
     sixteen-bit halves, each in a register of its own) is forgotten, the packed words remain */
  asm volatile("" : "+v"(next[0]), "+v"(next[1]), "+v"(next[2]), "+v"(next[3]), "+v"(done[0]),
                 "+v"(done[1]), "+v"(done[2]), "+v"(done[3]));
}

/*! \brief one row per workgroup, kHalfRowMinCols <= cols <= kHalfRowMaxCols. VEC as for
 *  SoftmaxAnyKernel. In place (dst == src) is safe: the row is read whole before it is written. */
template <bool VEC>
__global__ void __launch_bounds__(kHalfRowBlock, 4)  // four rows resident per CU
    SoftmaxHalfRowKernel(half::half_t *dst, uint32_t dstride, const half::half_t *src, uint32_t sstride,
                         uint32_t cols) {
  typedef half::half_t H;
  const int W = kHalfRowBlock / kWave;
  __shared__ MSHADOW_ALIGNED(16) uint16_t list[kHalfRowList];
  __shared__ uint32_t run_peak[kHalfRowPacks * W];
  __shared__ float run_total[kHalfRowPacks * W];
  __shared__ uint32_t run_count[kHalfRowPacks * W];
  __shared__ float wave_max[W];
  __shared__ uint32_t row_sum;
  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & (kWave - 1);
  const uint32_t wave = tid >> 6;
  const uint16_t *e = reinterpret_cast<const uint16_t *>(src) + static_cast<size_t>(blockIdx.x) * sstride;
  uint16_t *o = reinterpret_cast<uint16_t *>(dst) + static_cast<size_t>(blockIdx.x) * dstride;

  /* the row, and its maximum (`if (mmax < e[x]) mmax = e[x]` from e[0] on) */
  const uint32_t first = e[0];
  HalfPackWords v[kHalfRowPacks];
#pragma unroll
  for (int q = 0; q < kHalfRowPacks; ++q) {
    const uint32_t x = (q * kHalfRowBlock + tid) * kAnyTile;
    v[q] = HalfPackWords{first | (first << 16), first | (first << 16), first | (first << 16),
                         first | (first << 16)};
    if (x < cols) {
      if (VEC) {
        v[q] = *reinterpret_cast<const HalfPackWords *>(e + x);
      } else {
#pragma unroll
        for (int i = 0; i < kAnyTile; ++i) {
          if (x + i < cols) SetHalfBitsAt(v[q], i, e[x + i]);
        }
      }
    }
  }
  H h;
  h.half_ = static_cast<uint16_t>(first);
  float m = static_cast<float>(h);
#pragma unroll
  for (int q = 0; q < kHalfRowPacks; ++q) {
#pragma unroll
    for (int i = 0; i < kAnyTile; ++i) {
      h.half_ = static_cast<uint16_t>(HalfBitsAt(v[q], i));
      const float val = static_cast<float>(h);
      m = (m < val) ? val : m;
    }
  }
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const float other = WaveShuffleXor(m, d);
    m = (m < other) ? other : m;
  }
  if (lane == 0) wave_max[wave] = m;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < W; ++w) {
    const float other = wave_max[w];
    m = (m < other) ? other : m;
  }
  const H mmax = static_cast<H>(m);  // exact: m is one of the row's values
  /* the packed words are all that is kept of the row between the steps: without this the
     128 widened values of the maximum search stay in registers for the step below */
#pragma unroll
  for (int q = 0; q < kHalfRowPacks; ++q) {
    asm volatile("" : "+v"(v[q][0]), "+v"(v[q][1]), "+v"(v[q][2]), "+v"(v[q][3]));
  }

  /* the terms, in place of the logits; columns past the end of the row are zero terms */
#pragma unroll
  for (int q = 0; q < kHalfRowPacks; ++q) {
    const uint32_t x = (q * kHalfRowBlock + tid) * kAnyTile;
#pragma unroll
    for (int i = 0; i < kAnyTile; ++i) {
      h.half_ = static_cast<uint16_t>(HalfBitsAt(v[q], i));
      const H t = H(SoftmaxExp(h - mmax));
      /* whole packs: a pack is there or it is not (and 128 column numbers stay out of registers) */
      const bool there = VEC ? x < cols : x + i < cols;
      SetHalfBitsAt(v[q], i, there ? static_cast<uint32_t>(t.half_) : 0u);
    }
    OnePackAtATime(v[q], v[q + 1 < kHalfRowPacks ? q + 1 : 0]);
  }

  /* The list of the terms that count. The row is 64 runs of 512 terms in row order: run
     e = 4 q + w is what wave w holds of stretch q. A run's bound is made from the runs in
     front of it: the largest term so far, and a bound from the sums - every add, whether it
     changes the sum or not, returns at least (S + t) (1 - 2^-11), so behind a run of 512 adds
     the sum is at least ((sum in front) + (exact sum of the run)) (1 - 2^-11)^512.
     Three steps with a barrier behind each: every run's largest term and sum -> a table;
     every run's bound (all waves make the whole table, a lane per run) and count -> a table;
     every run's place in the list (a prefix over the table) and its entries. */
  const uint32_t nstretch = (cols + kHalfRowStretch - 1) / kHalfRowStretch;
  const float kKeep512 = 0.7787f;  // below (1 - 2^-11)^512 = 0.77875...
#pragma unroll
  for (int q = 0; q < kHalfRowPacks; ++q) {
    uint32_t peak = 0u;
    float total = 0.0f;
    if (static_cast<uint32_t>(q) < nstretch) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t lo = v[q][k] & 0x7fffu, hi = (v[q][k] >> 16) & 0x7fffu;
        peak = peak < lo ? lo : peak;
        peak = peak < hi ? hi : peak;
        total += static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(v[q][k] & 0xffffu)));
        total += static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(v[q][k] >> 16)));
      }
    }
    const uint32_t top = WaveInclusiveScanMaxU32(peak);
    const float all = WaveInclusiveScanF32(total);
    if (lane == kWave - 1) {
      run_peak[q * W + wave] = top;
      run_total[q * W + wave] = all;
    }
  }
  __syncthreads();
  /* lane e: the bounds in front of run e. The recurrence B' = (B + a) k is summed in closed
     form: B_e = k^e * sum over j < e of a_j k^-j (k^-63 is 7e6: no overflow). */
  uint32_t from_of_run;
  {
    const float a = run_total[lane] * 0.99975f;
    const uint32_t pk = run_peak[lane];
    const float up = __builtin_amdgcn_exp2f(static_cast<float>(lane) * 0.360900f);    // >= k^-e
    const float down = __builtin_amdgcn_exp2f(static_cast<float>(lane) * -0.360905f);  // <= k^e
    const float incl = WaveInclusiveScanF32(a * up);
    const float bound = (incl - a * up) * down * 0.999f;  // sum in front of run e, at least
    const uint32_t seen = WaveInclusiveScanMaxU32(pk);
    const uint32_t seen_before = static_cast<uint32_t>(
        __builtin_amdgcn_update_dpp(0, static_cast<int>(seen), 0x138, 0xf, 0xf, false));  // wave_shr:1
    /* the largest binary16 number not above the sum's bound (a NaN bound stays NaN: behind
       a NaN term nothing changes the sum) */
    const uint32_t sum_bits = H(bound * 0.999f).half_ & 0x7fffu;
    const uint32_t low = seen_before < sum_bits ? sum_bits : seen_before;
    from_of_run = HalfSignificantFrom(low);
  }
  uint32_t places[kHalfRowPacks / 2];  // per stretch: terms that count in the lanes below | own << 10
#pragma unroll
  for (int q = 0; q < kHalfRowPacks; ++q) {
    const uint32_t from = ReadLaneU32(from_of_run, q * W + static_cast<int>(wave));
    uint32_t mine = 0u;
#pragma unroll
    for (int i = 0; i < kAnyTile; ++i) mine += HalfBitsAt(v[q], i) >= from ? 1u : 0u;
    if (!(static_cast<uint32_t>(q) < nstretch)) mine = 0u;
    const uint32_t incl = WaveInclusiveScanU32(mine);
    if (lane == kWave - 1) run_count[q * W + wave] = incl;
    const uint32_t packed = (incl - mine) | (mine << 10);
    if (q & 1) {
      places[q >> 1] |= packed << 16;
    } else {
      places[q >> 1] = packed;
    }
  }
  __syncthreads();
  uint32_t count;
  bool fits;
  {
    const uint32_t c = run_count[lane];
    const uint32_t incl = WaveInclusiveScanU32(c);
    count = ReadLaneU32(incl, kWave - 1);
    fits = count <= static_cast<uint32_t>(kHalfRowList);
    const uint32_t first_of_run = incl - c;
    if (fits) {
#pragma unroll
      for (int q = 0; q < kHalfRowPacks; ++q) {
        const uint32_t from = ReadLaneU32(from_of_run, q * W + static_cast<int>(wave));
        const uint32_t packed = (places[q >> 1] >> ((q & 1) * 16)) & 0xffffu;
        uint32_t at = ReadLaneU32(first_of_run, q * W + static_cast<int>(wave)) + (packed & 0x3ffu);
        if ((packed >> 10) != 0u) {
#pragma unroll
          for (int i = 0; i < kAnyTile; ++i) {
            const uint32_t bits = HalfBitsAt(v[q], i);
            if (bits >= from) list[at++] = static_cast<uint16_t>(bits);
          }
        }
      }
    }
  }
  __syncthreads();
  /* One thread adds the list. Which wave it sits in rotates with the workgroup number: the
     chains of the rows that share a CU then run on different SIMDs (on one SIMD they would
     take turns: measured 11.4 ns per add for four of them, 5.6 ns for one). */
  const bool chain_thread = tid == (blockIdx.x % W) * kWave;
  if (fits) {
    if (chain_thread) {
      /* the whole row waits for this chain; the other waves on this SIMD (other rows' bulk
         steps) yield issue slots to it */
      __builtin_amdgcn_s_setprio(3);
      row_sum = ChainHalfList(H(0.0f).half_, list, count);
      __builtin_amdgcn_s_setprio(0);
    }
  } else {
    /* every term of a stretch, in row order, then the next stretch */
    uint32_t sum = H(0.0f).half_;
#pragma unroll
    for (int q = 0; q < kHalfRowPacks; ++q) {
      if (static_cast<uint32_t>(q) < nstretch) {
        *reinterpret_cast<HalfPackWords *>(list + tid * kAnyTile) = v[q];
        __syncthreads();
        if (chain_thread) {
          const uint32_t done = q * kHalfRowStretch;
          sum = ChainHalfList(sum, list, cols - done < static_cast<uint32_t>(kHalfRowStretch)
                                             ? cols - done : kHalfRowStretch);
        }
        __syncthreads();
      }
    }
    if (chain_thread) row_sum = sum;
  }
  __syncthreads();
  H sum;
  sum.half_ = static_cast<uint16_t>(row_sum);
#pragma unroll
  for (int q = 0; q < kHalfRowPacks; ++q) {
    const uint32_t x = (q * kHalfRowBlock + tid) * kAnyTile;
    if (x < cols) {
#pragma unroll
      for (int i = 0; i < kAnyTile; ++i) {
        h.half_ = static_cast<uint16_t>(HalfBitsAt(v[q], i));
        h /= sum;
        SetHalfBitsAt(v[q], i, h.half_);
      }
      if (q + 1 < kHalfRowPacks) OnePackAtATime(v[q], v[q + 1]);
      if (VEC) {
        *reinterpret_cast<HalfPackWords *>(o + x) = v[q];
      } else {
#pragma unroll
        for (int i = 0; i < kAnyTile; ++i) {
          if (x + i < cols) o[x + i] = static_cast<uint16_t>(HalfBitsAt(v[q], i));
        }
      }
    }
  }
}

/*! \brief which gradient: bit 0 label smoothing, bit 1 an ignored label (the values of
 *  MSHADOW_HIP_GRAD_SMOOTH / MSHADOW_HIP_GRAD_IGNORE) */
const int kAnyGradSmooth = 1;
const int kAnyGradIgnore = 2;

/*! \brief one element of SoftmaxGrad / SmoothSoftmaxGrad (mshadow/tensor_cpu-inl.h:286-455)
 *  with the host's expressions in the host's types: `p - 1.0f + alpha` and `p - smooth`
 *  round after every operation for half_t (its operators return half_t), are double
 *  arithmetic for double, and `smooth` = alpha / (classes - 1) is a float for every type */
template <typename DType, int FLAGS>
__device__ __forceinline__ DType GradElement(const DType &p, bool at_label, bool ignored,
                                             float alpha, float smooth) {
  if ((FLAGS & kAnyGradIgnore) && ignored) return DType(0.0f);
  if (FLAGS & kAnyGradSmooth) {
    if (at_label) return DType(p - 1.0f + alpha);
    return DType(p - smooth);
  }
  if (at_label) return DType(p - 1.0f);
  return p;
}

/*! \brief dst = the gradient FLAGS selects for probabilities src and labels label; a label
 *  outside the row marks no column. blockIdx.x = row, blockIdx.y = stretch of columns; a
 *  thread moves packs of kAnyTile elements. VEC as for SoftmaxAnyKernel. */
template <typename DType, bool VEC, int FLAGS>
__global__ void __launch_bounds__(kAnyBlock)
    SoftmaxGradAnyKernel(DType *dst, uint32_t dstride, const DType *src, uint32_t sstride,
                         const DType *label, uint32_t cols, int ignore_k, float alpha,
                         float smooth) {
  const uint32_t row = blockIdx.x;
  const int k = LabelIndex(label[row]);
  const bool ignored = (FLAGS & kAnyGradIgnore) && k == ignore_k;
  const DType *s = src + static_cast<size_t>(row) * sstride;
  DType *o = dst + static_cast<size_t>(row) * dstride;
  const uint32_t step = gridDim.y * kAnyBlock * kAnyTile;
  for (uint32_t x = (blockIdx.y * kAnyBlock + threadIdx.x) * kAnyTile; x < cols; x += step) {
    AnyPack<DType> v;
    LoadAnyPack<DType, VEC>(&v, s, x, cols, DType(0.0f));
    const uint32_t off = static_cast<uint32_t>(k) - x;  // wraps for k < x
    const bool label_here = k >= 0 && off < static_cast<uint32_t>(kAnyTile);
    if (FLAGS != 0 || label_here) {
#pragma unroll
      for (int i = 0; i < kAnyTile; ++i) {
        v.v[i] = GradElement<DType, FLAGS>(v.v[i], label_here && static_cast<uint32_t>(i) == off,
                                           ignored, alpha, smooth);
      }
    }
    StoreAnyPack<DType, VEC>(o, x, cols, v);
  }
}

/* ---- tensors of three dimensions (d0, d1, d2): the softmax runs over the middle one
 * (mshadow/tensor_cpu-inl.h:466-488). Element (y, x, n) is at (y * d1 + x) * stride + n. */
const int kAny3dBlock = 256;

/*! \brief one thread per (y, n), neighbouring threads neighbouring n (coalesced): the
 *  thread walks x three times, exactly as the host loop does - maximum, terms stored and
 *  summed left to right in DType, quotients. In place (dst == src) is safe: a thread reads
 *  and writes its own column only. */
template <typename DType>
__global__ void __launch_bounds__(kAny3dBlock)
    Softmax3dAnyKernel(DType *dst, uint32_t dstride, const DType *src, uint32_t sstride,
                       uint32_t d0, uint32_t d1, uint32_t d2) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * kAny3dBlock + threadIdx.x;
  if (idx >= static_cast<size_t>(d0) * d2) return;
  const uint32_t y = static_cast<uint32_t>(idx / d2);
  const uint32_t n = static_cast<uint32_t>(idx - static_cast<size_t>(y) * d2);
  const DType *s = src + static_cast<size_t>(y) * d1 * sstride + n;
  DType *o = dst + static_cast<size_t>(y) * d1 * dstride + n;
  DType mmax = s[0];
  for (uint32_t x = 1; x < d1; ++x) {
    const DType e = s[static_cast<size_t>(x) * sstride];
    if (mmax < e) mmax = e;
  }
  DType sum = DType(0.0f);
  for (uint32_t x = 0; x < d1; ++x) {
    const DType t = DType(SoftmaxExp(DType(s[static_cast<size_t>(x) * sstride] - mmax)));
    o[static_cast<size_t>(x) * dstride] = t;
    ChainAdd(sum, t);
  }
  for (uint32_t x = 0; x < d1; ++x) {
    DType t = o[static_cast<size_t>(x) * dstride];
    t /= sum;
    o[static_cast<size_t>(x) * dstride] = t;
  }
}

/*! \brief one thread per element; label (y, n) at y * lstride + n */
template <typename DType, int FLAGS>
__global__ void __launch_bounds__(kAny3dBlock)
    SoftmaxGrad3dAnyKernel(DType *dst, uint32_t dstride, const DType *src, uint32_t sstride,
                           const DType *label, uint32_t lstride, uint32_t d0, uint32_t d1,
                           uint32_t d2, int ignore_k, float alpha, float smooth) {
  const size_t total = static_cast<size_t>(d0) * d1 * d2;
  for (size_t idx = static_cast<size_t>(blockIdx.x) * kAny3dBlock + threadIdx.x; idx < total;
       idx += static_cast<size_t>(gridDim.x) * kAny3dBlock) {
    const size_t row = idx / d2;  // y * d1 + x
    const uint32_t n = static_cast<uint32_t>(idx - row * d2);
    const uint32_t y = static_cast<uint32_t>(row / d1);
    const uint32_t x = static_cast<uint32_t>(row - static_cast<size_t>(y) * d1);
    const int k = LabelIndex(label[static_cast<size_t>(y) * lstride + n]);
    const bool ignored = (FLAGS & kAnyGradIgnore) && k == ignore_k;
    dst[row * dstride + n] = GradElement<DType, FLAGS>(src[row * sstride + n],
                                                       static_cast<int>(x) == k, ignored, alpha,
                                                       smooth);
  }
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_SOFTMAX_ANY_H_
