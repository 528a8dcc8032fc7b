/*
 * Row scatter / gather by an index vector: AddTakeGrad, AddTakeGradLargeBatch, IndexFill
 * (mshadow/tensor_cpu-inl.h:497-528; the reference's GPU versions are
 * cuda/tensor_gpu-inl.cuh:599-782).
 *
 * The CPU functions walk the index vector front to back, so a destination row that is
 * named several times receives its additions in index order (a float sum depends on it)
 * and, for IndexFill, keeps the LAST source row written to it. To reproduce that without
 * a sort or a workspace, every destination row has one owner wave that applies the entries
 * naming it in index order, the lanes spread over the columns; nothing else touches the row,
 * so there is no atomic and no race. The sixteen waves of a workgroup share one scan of the
 * index vector (RowsByIndexKernel).
 */
#ifndef MSHADOW_AMD_CSRC_ROW_KERNELS_H_
#define MSHADOW_AMD_CSRC_ROW_KERNELS_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mshadow/hip/kernels/common.h>

namespace mshadow_hipk {


/*! \brief entry y of an index vector stored as int32 or as float (truncated like a label) */
template <bool IS_INT>
__device__ __forceinline__ int IndexAt(const void *index, int y) {
  return IS_INT ? static_cast<const int32_t *>(index)[y]
                : static_cast<int>(static_cast<const float *>(index)[y]);
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

/*! \brief the row operation OP for y = 0 .. n_index-1 in order.
 *  a workgroup owns 16 * rows_per_wave consecutive destination rows and scans the index
 *  vector once, 1024 entries at a time. The entries of a chunk that fall into its rows are
 *  compacted, in index order, into a list in LDS (a ballot per wave and a prefix over the
 *  waves); each wave then applies the listed entries that name its own rows_per_wave rows,
 *  in list order, the lanes spread over the columns. Rows of different waves are disjoint and
 *  chunks follow each other, so every row receives its additions in index order - with no
 *  atomic, no sort and no workspace. Scan work is (rows / rows per workgroup) * entries / 64
 *  wave-steps. VEC4: rows are whole aligned 16-byte packs. */
template <bool IS_INT, int OP, bool VEC4>
__global__ void __launch_bounds__(kTakeBlock)
    RowsByIndexKernel(float *dst, int dstride, int k_rows, int rows_per_wave,
                           const void *rows_of, const void *from_of, int n_index, const float *src,
                           int sstride, int cols) {
  typedef float F4 __attribute__((ext_vector_type(4)));
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
  if (static_cast<int>(threadIdx.x) < n_index) fetched = IndexAt<IS_INT>(rows_of, threadIdx.x);
  for (int c0 = 0; c0 < n_index; c0 += kTakeBlock, buf ^= 1) {
    const int y = c0 + static_cast<int>(threadIdx.x);
    int r = y < n_index ? fetched : -1;
    if (CLAMP && y < n_index) r = r <= 0 ? 0 : (r >= k_rows ? k_rows - 1 : r);
    if (y + kTakeBlock < n_index) fetched = IndexAt<IS_INT>(rows_of, y + kTakeBlock);
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
        const int from = FROM_ENTRY ? entry : IndexAt<IS_INT>(from_of, entry);
        const float *in = src + static_cast<size_t>(from) * sstride;
        float *out = dst + static_cast<size_t>(row) * dstride;
        if (VEC4) {
          /* four packs per lane are fetched from both rows before any is written: within one
             row the fetches do not wait for each other's stores */
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
        } else {
          for (int x = lane; x < cols; x += 64) out[x] = OP == kFill ? in[x] : out[x] + in[x];
        }
      }
    }
  }
}

}  // namespace mshadow_hipk
#endif  // MSHADOW_AMD_CSRC_ROW_KERNELS_H_
