/*
 * Row scatter / gather by an index vector: AddTakeGrad, AddTakeGradLargeBatch, IndexFill
 * (mshadow/tensor_cpu-inl.h:497-528; the reference's GPU versions are
 * cuda/tensor_gpu-inl.cuh:599-782), for any element type and any index type.
 *
 * The CPU functions walk the index vector front to back, so a destination row that is
 * named several times receives its additions in index order (a floating-point sum depends
 * on it) and, for IndexFill, keeps the LAST source row written to it. To reproduce that
 * without a sort or a workspace, every destination row has one owner wave that applies the
 * entries naming it in index order, the lanes spread over the columns; nothing else touches
 * the row, so there is no atomic and no race. The sixteen waves of a workgroup share one
 * scan of the index vector. Additions are made in the element type's own arithmetic
 * (half_t: widen, add in float, round back - one rounding per addition, as on the host).
 */
#ifndef MSHADOW_HIP_KERNELS_ROWS_BY_INDEX_H_
#define MSHADOW_HIP_KERNELS_ROWS_BY_INDEX_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../half.h"
#include "./common.h"

namespace mshadow {
namespace hip {

/*! \brief entry y of an index vector as the host reads it: `int j = index[y]`
 *  (a floating-point entry is truncated like a label, half_t through float) */
template <typename IndexType>
__device__ __forceinline__ int IndexAt(const IndexType *index, int y) {
  return static_cast<int>(index[y]);
}
__device__ __forceinline__ int IndexAt(const half::half_t *index, int y) {
  return static_cast<int>(static_cast<float>(index[y]));
}

const int kTakeBlock = 1024;  // sixteen waves share one scan of the index vector

/*! \brief what the three functions do to a destination row for entry y, front to back */
enum RowOp {
  kTakeGrad = 0,       //!< dst[clamp(index[y])] += src[y]                      (AddTakeGrad)
  kTakeGradSorted = 1, //!< dst[sorted[y]] += src[index[y]], rows outside the table skipped
                       //!< (AddTakeGradLargeBatch; also right when `sorted` is not sorted)
  kFill = 2            //!< dst[index[y]] = src[y], rows outside the table skipped: of several
                       //!< entries naming one row the last one counts          (IndexFill)
};

/*! \brief one wave applies one source row to one destination row */
template <typename DType, int OP, bool VEC4>
struct RowApply {
  __device__ __forceinline__ static void Run(DType *out, const DType *in, int cols, int lane) {
    for (int x = lane; x < cols; x += 64) {
      if (OP == kFill) {
        out[x] = in[x];
      } else {
        out[x] += in[x];
      }
    }
  }
};
/*! \brief float rows of whole aligned 16-byte packs: four packs per lane are fetched from
 *  both rows before any is written, so that within one row the fetches do not wait for each
 *  other's stores */
template <int OP>
struct RowApply<float, OP, true> {
  __device__ __forceinline__ static void Run(float *out, const float *in, int cols, int lane) {
    typedef float F4 __attribute__((ext_vector_type(4)));
    for (int x0 = lane * 4; x0 < cols; x0 += 1024) {
      F4 a[4], c[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int x = x0 + k * 256;
        if (x < cols) {
          if (OP != kFill) a[k] = *reinterpret_cast<const F4 *>(out + x);
          c[k] = __builtin_nontemporal_load(reinterpret_cast<const F4 *>(in + x));
        }
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int x = x0 + k * 256;
        if (x < cols) *reinterpret_cast<F4 *>(out + x) = OP == kFill ? c[k] : a[k] + c[k];
      }
    }
  }
};

/*! \brief the row operation OP for y = 0 .. n_index-1 in order.
 *  a workgroup owns 16 * rows_per_wave consecutive destination rows and scans the index
 *  vector once, 1024 entries at a time. The entries of a chunk that fall into its rows are
 *  compacted, in index order, into a list in LDS (a ballot per wave and a prefix over the
 *  waves); each wave then applies the listed entries that name its own rows_per_wave rows,
 *  in list order, the lanes spread over the columns. Rows of different waves are disjoint and
 *  chunks follow each other, so every row receives its additions in index order - with no
 *  atomic, no sort and no workspace. Scan work is (rows / rows per workgroup) * entries / 64
 *  wave-steps. VEC4 (float only): rows are whole aligned 16-byte packs. */
template <typename IndexType, typename DType, int OP, bool VEC4>
__global__ void __launch_bounds__(kTakeBlock)
    RowsByIndexKernel(DType *dst, int dstride, int k_rows, int rows_per_wave,
                      const IndexType *rows_of, const IndexType *from_of, int n_index,
                      const DType *src, int sstride, int cols) {
  const bool CLAMP = OP == kTakeGrad;
  const bool FROM_ENTRY = OP != kTakeGradSorted;
  const int W = kTakeBlock / 64;
  __shared__ int list_y[2][kTakeBlock];
  __shared__ int list_r[2][kTakeBlock];
  __shared__ int wave_count[2][W];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long long block_first = static_cast<long long>(blockIdx.x) * W * rows_per_wave;
  const int b0 = static_cast<int>(block_first);
  const int b1 = block_first + W * rows_per_wave < k_rows ? b0 + W * rows_per_wave : k_rows;
  const int my0 = b0 + wave * rows_per_wave;
  const int my1 = my0 + rows_per_wave < b1 ? my0 + rows_per_wave : b1;
  int buf = 0;
  /* the entry of the next chunk is fetched while the current chunk is handled */
  int fetched = -1;
  if (static_cast<int>(threadIdx.x) < n_index) fetched = IndexAt(rows_of, threadIdx.x);
  for (int c0 = 0; c0 < n_index; c0 += kTakeBlock, buf ^= 1) {
    const int y = c0 + static_cast<int>(threadIdx.x);
    int r = y < n_index ? fetched : -1;
    if (CLAMP && y < n_index) r = r <= 0 ? 0 : (r >= k_rows ? k_rows - 1 : r);
    if (y + kTakeBlock < n_index) fetched = IndexAt(rows_of, y + kTakeBlock);
    const bool hit = r >= b0 && r < b1;
    const unsigned long long mask = __ballot(hit);
    if (lane == 0) wave_count[buf][wave] = __popcll(mask);
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      const int c = wave_count[buf][w];
      before += w < wave ? c : 0;
      total += c;
    }
    if (total == 0) continue;  // uniform: every wave read the same counts
    if (hit) {
      const int pos = before + __popcll(mask & ((1ull << lane) - 1ull));
      list_y[buf][pos] = y;
      list_r[buf][pos] = r;
    }
    __syncthreads();
    for (int i0 = 0; i0 < total; i0 += 64) {
      const int e = i0 + lane;
      const int er = e < total ? list_r[buf][e] : -1;
      const int ey = e < total ? list_y[buf][e] : 0;
      unsigned long long mine = __ballot(er >= my0 && er < my1);
      while (mine != 0ull) {
        const int b = __ffsll(static_cast<long long>(mine)) - 1;
        mine &= mine - 1ull;
        const int row = __shfl(er, b);
        const int entry = __shfl(ey, b);
        const int from = FROM_ENTRY ? entry : IndexAt(from_of, entry);
        RowApply<DType, OP, VEC4>::Run(dst + static_cast<size_t>(row) * dstride,
                                       src + static_cast<size_t>(from) * sstride, cols, lane);
      }
    }
  }
}

/*! \brief grid and rows per wave for a table of k_rows rows: about as many workgroups as the
 *  machine holds at once (two of these per CU), each owning a run of destination rows */
inline void RowsByIndexGrid(int k_rows, unsigned *grid, int *rows_per_wave) {
  const int kWavesPerBlock = kTakeBlock / 64;
  const int rows_per_block_wanted = (k_rows + 511) / 512;
  *rows_per_wave = (rows_per_block_wanted + kWavesPerBlock - 1) / kWavesPerBlock;
  const int rows_per_block = *rows_per_wave * kWavesPerBlock;
  *grid = static_cast<unsigned>((k_rows + rows_per_block - 1) / rows_per_block);
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_ROWS_BY_INDEX_H_
