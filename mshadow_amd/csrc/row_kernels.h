/*
 * Row scatter / gather by an index vector: AddTakeGrad, AddTakeGradLargeBatch, IndexFill
 * (mshadow/tensor_cpu-inl.h:497-528; the reference's GPU versions are
 * cuda/tensor_gpu-inl.cuh:599-782).
 *
 * The CPU functions walk the index vector front to back, so a destination row that is
 * named several times receives its additions in index order (a float sum depends on it)
 * and, for IndexFill, keeps the LAST source row written to it. To reproduce that without
 * a sort or a workspace, one wave owns one destination row: it scans the whole index
 * vector 64 entries at a time (coalesced), finds the entries that name its row with a
 * ballot, and applies them in order, the lanes spread over the columns. Work is
 * rows * entries / 64 wave-steps - fine for embedding-sized problems, and nothing else
 * touches the row, so there is no atomic and no race.
 */
#ifndef MSHADOW_AMD_CSRC_ROW_KERNELS_H_
#define MSHADOW_AMD_CSRC_ROW_KERNELS_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mshadow/hip/kernels/common.h>

namespace mshadow_hipk {

const int kRowBlock = 256;  // four destination rows per workgroup

/*! \brief entry y of an index vector stored as int32 or as float (truncated like a label) */
template <bool IS_INT>
__device__ __forceinline__ int IndexAt(const void *index, int y) {
  return IS_INT ? static_cast<const int32_t *>(index)[y]
                : static_cast<int>(static_cast<const float *>(index)[y]);
}

/*! \brief dst[row(y)] += src[from(y)] for y = 0 .. n_index-1 in order.
 *  CLAMP: row(y) = index[y] clamped into [0, k_rows) and from(y) = y    (AddTakeGrad);
 *  else:  row(y) = sorted[y] and from(y) = index[y]                   (AddTakeGradLargeBatch,
 *  which therefore also gives the reference's result when `sorted` is not sorted). */
template <bool IS_INT, bool CLAMP>
__global__ void __launch_bounds__(kRowBlock)
    AddTakeGradKernel(float *dst, int dstride, int k_rows, const void *rows_of, const void *from_of,
                      int n_index, const float *src, int sstride, int cols) {
  const int lane = threadIdx.x & 63;
  const int j = blockIdx.x * (kRowBlock / 64) + (threadIdx.x >> 6);
  if (j >= k_rows) return;
  float *out = dst + static_cast<size_t>(j) * dstride;
  for (int y0 = 0; y0 < n_index; y0 += 64) {
    const int y = y0 + lane;
    int r = -1;
    if (y < n_index) {
      r = IndexAt<IS_INT>(rows_of, y);
      if (CLAMP) r = r <= 0 ? 0 : (r >= k_rows ? k_rows - 1 : r);
    }
    unsigned long long hits = __ballot(r == j);
    while (hits != 0ull) {
      const int b = __ffsll(static_cast<long long>(hits)) - 1;
      hits &= hits - 1ull;
      const int from = CLAMP ? y0 + b : IndexAt<IS_INT>(from_of, y0 + b);
      const float *in = src + static_cast<size_t>(from) * sstride;
      for (int x = lane; x < cols; x += 64) out[x] = out[x] + in[x];
    }
  }
}

/*! \brief the same result with one wave per ENTRY of the index vector instead of one per
 *  destination row, for tables with more rows than there are entries: the wave of entry y
 *  looks for an earlier entry naming the same row and retires if there is one; the wave of
 *  a row's first entry then applies all of that row's entries in order. Work is about
 *  entries^2 / 64 wave-steps, independent of the number of rows. */
template <bool IS_INT, bool CLAMP>
__global__ void __launch_bounds__(kRowBlock)
    AddTakeGradByEntryKernel(float *dst, int dstride, int k_rows, const void *rows_of,
                             const void *from_of, int n_index, const float *src, int sstride,
                             int cols) {
  const int lane = threadIdx.x & 63;
  const int me = blockIdx.x * (kRowBlock / 64) + (threadIdx.x >> 6);
  if (me >= n_index) return;
  int j = IndexAt<IS_INT>(rows_of, me);
  if (CLAMP) j = j <= 0 ? 0 : (j >= k_rows ? k_rows - 1 : j);
  if (j < 0 || j >= k_rows) return;
  float *out = dst + static_cast<size_t>(j) * dstride;
  for (int y0 = 0; y0 < n_index; y0 += 64) {
    const int y = y0 + lane;
    int r = -1;
    if (y < n_index) {
      r = IndexAt<IS_INT>(rows_of, y);
      if (CLAMP) r = r <= 0 ? 0 : (r >= k_rows ? k_rows - 1 : r);
    }
    unsigned long long hits = __ballot(r == j);
    if (y0 <= me && hits != 0ull) {
      /* the first entry of the row, at or before mine, is in this chunk */
      if (y0 + __ffsll(static_cast<long long>(hits)) - 1 != me) return;  // not the row's first entry
    }
    if (y0 + 63 < me) continue;  // still in front of my entry: nothing to apply yet
    while (hits != 0ull) {
      const int b = __ffsll(static_cast<long long>(hits)) - 1;
      hits &= hits - 1ull;
      const int from = CLAMP ? y0 + b : IndexAt<IS_INT>(from_of, y0 + b);
      const float *in = src + static_cast<size_t>(from) * sstride;
      for (int x = lane; x < cols; x += 64) out[x] = out[x] + in[x];
    }
  }
}

/*! \brief IndexFill by entry: the wave of entry y copies its row unless a later entry names
 *  the same destination */
template <bool IS_INT>
__global__ void __launch_bounds__(kRowBlock)
    IndexFillByEntryKernel(float *dst, int dstride, int k_rows, const void *index, int n_index,
                           const float *src, int sstride, int cols) {
  const int lane = threadIdx.x & 63;
  const int me = blockIdx.x * (kRowBlock / 64) + (threadIdx.x >> 6);
  if (me >= n_index) return;
  const int j = IndexAt<IS_INT>(index, me);
  if (j < 0 || j >= k_rows) return;
  for (int y0 = (me / 64) * 64; y0 < n_index; y0 += 64) {
    const int y = y0 + lane;
    const bool later = y > me && y < n_index && IndexAt<IS_INT>(index, y) == j;
    if (__ballot(later) != 0ull) return;
  }
  const float *in = src + static_cast<size_t>(me) * sstride;
  float *out = dst + static_cast<size_t>(j) * dstride;
  for (int x = lane; x < cols; x += 64) out[x] = in[x];
}

/*! \brief dst[index[y]] = src[y]; of several entries naming one row the last one counts */
template <bool IS_INT>
__global__ void __launch_bounds__(kRowBlock)
    IndexFillKernel(float *dst, int dstride, int k_rows, const void *index, int n_index,
                    const float *src, int sstride, int cols) {
  const int lane = threadIdx.x & 63;
  const int j = blockIdx.x * (kRowBlock / 64) + (threadIdx.x >> 6);
  if (j >= k_rows) return;
  int last = -1;
  for (int y0 = 0; y0 < n_index; y0 += 64) {
    const int y = y0 + lane;
    const bool hit = y < n_index && IndexAt<IS_INT>(index, y) == j;
    const unsigned long long hits = __ballot(hit);
    if (hits != 0ull) last = y0 + 63 - __clzll(static_cast<long long>(hits));
  }
  if (last < 0) return;
  const float *in = src + static_cast<size_t>(last) * sstride;
  float *out = dst + static_cast<size_t>(j) * dstride;
  for (int x = lane; x < cols; x += 64) out[x] = in[x];
}

}  // namespace mshadow_hipk
#endif  // MSHADOW_AMD_CSRC_ROW_KERNELS_H_
