/*
 * Permutation of the axes of a dense tensor of 32-bit elements: dst axis i is src axis
 * axes[i]. This is what `dst = transpose(src, axes)` and `dst = swapaxis<a1, a2>(src)`
 * compute (mshadow/extension/transpose.h:24-88, swapaxis.h:20-106 of the reference, which
 * evaluate them element by element through the generic map kernel).
 *
 * On the host the problem is first reduced: axes of length 1 are dropped and axes that
 * stay neighbours in the same order are merged, so NCHW -> NHWC becomes a batch of 2-D
 * transposes (n, c, h*w) -> (n, h*w, c). Then
 *  - if the last axis stays last, rows are permuted: one thread per 16 bytes (or per
 *    element), the source row found by taking the destination row number apart;
 *  - otherwise the source's last axis (extent L) lands on some other destination axis and
 *    the destination's last axis (extent A) comes from some other source axis: the two span
 *    a plane that is moved in 64 x 64 tiles through LDS, read along L and written along A,
 *    so that both sides are coalesced. The remaining axes are batch indices.
 * Pure data movement: bit-exact. HBM-bound, 2 * 4 bytes per element.
 *
 * Also here: the fill of a 2-D view with one 32-bit pattern (`tensor = scalar`) and the
 * device-to-device copy of a pitched 2-D view (`Copy(Tensor<gpu>, Tensor<gpu>)`).
 */
#include <algorithm>

#include <mshadow/core/fastdiv.h>
#include <mshadow/hip/kernels/common.h>

#include "./abi_common.h"

using mshadow::FastDivU32;
using mshadow_abi::AfterLaunch;
using mshadow_abi::AsStream;

namespace {

const int kMaxAxes = 6;
const int kTile = 64;
const int kPermuteBlock = 256;

/*! \brief the batch axes of the reduced problem: how to take a batch number apart and what
 *  each digit is worth in the source and in the destination */
struct BatchAxes {
  int count;
  FastDivU32 extent[kMaxAxes];
  uint32_t src_step[kMaxAxes];
  uint32_t dst_step[kMaxAxes];
  __device__ __forceinline__ void Offsets(uint32_t batch, uint32_t *src_off, uint32_t *dst_off) const {
    uint32_t s = 0, d = 0;
    for (int k = count - 1; k >= 0; --k) {
      const uint32_t q = extent[k].Div(batch);
      const uint32_t digit = batch - q * extent[k].div;
      s += digit * src_step[k];
      d += digit * dst_step[k];
      batch = q;
    }
    *src_off = s;
    *dst_off = d;
  }
};

/*! \brief one 64 x 64 tile of the (A, L) plane per workgroup: src[batch][a][l] at
 *  a * src_step_a + l, dst[batch][l][a] at l * dst_step_l + a */
__global__ void __launch_bounds__(kPermuteBlock)
    PermuteTileKernel(uint32_t *dst, const uint32_t *src, uint32_t extent_a, uint32_t extent_l,
                      uint32_t src_step_a, uint32_t dst_step_l, FastDivU32 tiles_a,
                      FastDivU32 tiles_l, BatchAxes batch_axes) {
  __shared__ uint32_t tile[kTile][kTile + 1];
  const uint32_t block = mshadow::hip::StripOfBlock(blockIdx.x, gridDim.x);
  const uint32_t rest = tiles_l.Div(block);
  const uint32_t tl = block - rest * tiles_l.div;
  const uint32_t batch = tiles_a.Div(rest);
  const uint32_t ta = rest - batch * tiles_a.div;
  uint32_t src_off, dst_off;
  batch_axes.Offsets(batch, &src_off, &dst_off);
  const uint32_t tx = threadIdx.x % kTile, ty = threadIdx.x / kTile;
  const int kRowsPerPass = kPermuteBlock / kTile;
  {
    const uint32_t l = tl * kTile + tx;
    const uint32_t *from = src + src_off + l;
#pragma unroll
    for (int r = 0; r < kTile; r += kRowsPerPass) {
      const uint32_t a = ta * kTile + r + ty;
      if (a < extent_a && l < extent_l) {
        tile[r + ty][tx] = __builtin_nontemporal_load(from + static_cast<size_t>(a) * src_step_a);
      }
    }
  }
  __syncthreads();
  {
    const uint32_t a = ta * kTile + tx;
    uint32_t *to = dst + dst_off + a;
#pragma unroll
    for (int r = 0; r < kTile; r += kRowsPerPass) {
      const uint32_t l = tl * kTile + r + ty;
      if (a < extent_a && l < extent_l) {
        __builtin_nontemporal_store(tile[tx][r + ty], to + static_cast<size_t>(l) * dst_step_l);
      }
    }
  }
}

/*! \brief the same tile with 128-bit global accesses on both sides (extents, steps and
 *  offsets are multiples of four words, pointers 16-byte aligned). A thread moves four
 *  adjacent words of a row; the transposition happens in the word-wise LDS accesses, whose
 *  row pitch of 65 words spreads the 64 lanes over all banks. */
__global__ void __launch_bounds__(kPermuteBlock)
    PermuteTileVecKernel(uint32_t *dst, const uint32_t *src, uint32_t extent_a, uint32_t extent_l,
                         uint32_t src_step_a, uint32_t dst_step_l, FastDivU32 tiles_a,
                         FastDivU32 tiles_l, BatchAxes batch_axes) {
  typedef uint32_t Vec4 __attribute__((ext_vector_type(4)));
  __shared__ uint32_t tile[kTile][kTile + 1];
  const uint32_t block = mshadow::hip::StripOfBlock(blockIdx.x, gridDim.x);
  const uint32_t rest = tiles_l.Div(block);
  const uint32_t tl = block - rest * tiles_l.div;
  const uint32_t batch = tiles_a.Div(rest);
  const uint32_t ta = rest - batch * tiles_a.div;
  uint32_t src_off, dst_off;
  batch_axes.Offsets(batch, &src_off, &dst_off);
  const int kLanesPerRow = kTile / 4;                       // 16 threads cover a row of the tile
  const int kRowsPerPass = kPermuteBlock / kLanesPerRow;    // 16 rows per pass
  const uint32_t tx = (threadIdx.x % kLanesPerRow) * 4, ty = threadIdx.x / kLanesPerRow;
  {
    const uint32_t l = tl * kTile + tx;
    const uint32_t *from = src + src_off + l;
    Vec4 got[kTile / kRowsPerPass];
#pragma unroll
    for (int r = 0; r < kTile; r += kRowsPerPass) {
      const uint32_t a = ta * kTile + r + ty;
      if (a < extent_a && l < extent_l) {
        got[r / kRowsPerPass] = __builtin_nontemporal_load(
            reinterpret_cast<const Vec4 *>(from + static_cast<size_t>(a) * src_step_a));
      }
    }
#pragma unroll
    for (int r = 0; r < kTile; r += kRowsPerPass) {
      const Vec4 v = got[r / kRowsPerPass];
      tile[r + ty][tx + 0] = v.x;
      tile[r + ty][tx + 1] = v.y;
      tile[r + ty][tx + 2] = v.z;
      tile[r + ty][tx + 3] = v.w;
    }
  }
  __syncthreads();
  {
    const uint32_t a = ta * kTile + tx;
    uint32_t *to = dst + dst_off + a;
#pragma unroll
    for (int r = 0; r < kTile; r += kRowsPerPass) {
      const uint32_t l = tl * kTile + r + ty;
      Vec4 v;
      v.x = tile[tx + 0][r + ty];
      v.y = tile[tx + 1][r + ty];
      v.z = tile[tx + 2][r + ty];
      v.w = tile[tx + 3][r + ty];
      if (a < extent_a && l < extent_l) {
        __builtin_nontemporal_store(v, reinterpret_cast<Vec4 *>(to + static_cast<size_t>(l) * dst_step_l));
      }
    }
  }
}

/*! \brief the last axis stays: destination row `row` is source row Offsets(row); WORDS
 *  32-bit words per thread (4 when rows are made of whole aligned 16-byte packs) */
template <int WORDS>
__global__ void __launch_bounds__(kPermuteBlock)
    PermuteRowsKernel(uint32_t *dst, const uint32_t *src, uint32_t rows, uint32_t cols,
                      FastDivU32 packs_per_row, BatchAxes row_axes) {
  typedef uint32_t Vec __attribute__((ext_vector_type(WORDS)));
  const uint32_t total = rows * packs_per_row.div;
  const uint32_t step = gridDim.x * kPermuteBlock;
  const uint32_t block = mshadow::hip::StripOfBlock(blockIdx.x, gridDim.x);
  for (uint32_t p = block * kPermuteBlock + threadIdx.x; p < total; p += step) {
    const uint32_t row = packs_per_row.Div(p);
    const uint32_t x = (p - row * packs_per_row.div) * WORDS;
    uint32_t src_off, dst_off;
    row_axes.Offsets(row, &src_off, &dst_off);
    const Vec v = __builtin_nontemporal_load(reinterpret_cast<const Vec *>(src + src_off + x));
    __builtin_nontemporal_store(v, reinterpret_cast<Vec *>(dst + static_cast<size_t>(row) * cols + x));
  }
}

/*! \brief every element of a pitched 2-D view set to one 32-bit pattern; WORDS words per
 *  store (4 when rows are made of whole aligned 16-byte packs) */
template <int WORDS>
__global__ void __launch_bounds__(kPermuteBlock)
    FillKernel(uint32_t *dst, uint32_t stride, uint32_t rows, uint32_t packs_per_row,
               FastDivU32 div_ppr, uint32_t bits) {
  typedef uint32_t Vec __attribute__((ext_vector_type(WORDS)));
  Vec v;
#pragma unroll
  for (int k = 0; k < WORDS; ++k) v[k] = bits;
  const uint32_t total = rows * packs_per_row;
  const uint32_t step = gridDim.x * kPermuteBlock;
  for (uint32_t i = blockIdx.x * kPermuteBlock + threadIdx.x; i < total; i += step) {
    const uint32_t y = div_ppr.Div(i);
    __builtin_nontemporal_store(
        v, reinterpret_cast<Vec *>(dst + static_cast<size_t>(y) * stride + (i - y * packs_per_row) * WORDS));
  }
}

/*! \brief rows of `per_row` units of type T copied between two pitched views (pitches in
 *  units), UNROLL units per thread with all loads issued before the first store; FLAT: both
 *  views are dense, the copy is one run and no row number is ever computed. The data passes
 *  through once: streaming loads and stores. */
template <typename T, int UNROLL, bool FLAT>
__global__ void __launch_bounds__(kPermuteBlock)
    CopyRowsKernel(T *dst, size_t dpitch, const T *src, size_t spitch, uint32_t total,
                   uint32_t per_row, FastDivU32 div_per_row) {
  const uint32_t base = blockIdx.x * (kPermuteBlock * UNROLL) + threadIdx.x;
  T v[UNROLL];
  size_t to[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const uint32_t p = base + u * kPermuteBlock;
    size_t from = p;
    to[u] = p;
    if (!FLAT) {
      const uint32_t y = div_per_row.Div(p);
      const uint32_t x = p - y * per_row;
      from = static_cast<size_t>(y) * spitch + x;
      to[u] = static_cast<size_t>(y) * dpitch + x;
    }
    if (p < total) v[u] = __builtin_nontemporal_load(src + from);
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    if (base + u * kPermuteBlock < total) __builtin_nontemporal_store(v[u], dst + to[u]);
  }
}

/* 16 bytes per thread, whatever the unit: 8192x32000 floats by 16-byte units in 321 us with one
   unit per thread, 345 us with four, 500 us with eight (MI355X) */
/*! \brief rows whose width, pitches or addresses are multiples of 4 but not of 16 bytes: still
 *  16 bytes per thread - such accesses need no alignment here -, the last pack of a row moved
 *  back so that it ends with the row (it overlaps its neighbour; both store the same bytes).
 *  Rows of 16 bytes or more. 8192 rows of 127,960 bytes at a pitch of 128,000: 0.78 of the HBM
 *  peak against 0.75 by 8-byte units. */
__global__ void __launch_bounds__(kPermuteBlock)
    CopyRowsAnywhereKernel(char *dst, size_t dpitch, const char *src, size_t spitch, uint32_t total,
                           uint32_t packs_per_row, uint32_t width, FastDivU32 div_ppr) {
  typedef uint32_t Vec4 __attribute__((ext_vector_type(4)));
  typedef Vec4 Loose __attribute__((aligned(4)));
  const uint32_t p = blockIdx.x * kPermuteBlock + threadIdx.x;
  if (p >= total) return;
  const uint32_t y = div_ppr.Div(p);
  uint32_t x = (p - y * packs_per_row) * 16u;
  x = x + 16u <= width ? x : width - 16u;
  const Vec4 v = __builtin_nontemporal_load(reinterpret_cast<const Loose *>(src + static_cast<size_t>(y) * spitch + x));
  __builtin_nontemporal_store(v, reinterpret_cast<Loose *>(dst + static_cast<size_t>(y) * dpitch + x));
}

template <typename T>
struct CopyUnroll {
  static const int value = sizeof(T) >= 16 ? 1 : 16 / sizeof(T);
};
const int kCopyMaxUnroll = 4;
const uint32_t kCopyMaxUnits = (1u << 31) - kPermuteBlock * kCopyMaxUnroll;  // per launch

template <typename T>
void LaunchCopyRows(void *dst, size_t dpitch_bytes, const void *src, size_t spitch_bytes,
                    size_t width_bytes, size_t rows, hipStream_t s) {
  const size_t unit = sizeof(T);
  const int kCopyUnroll = CopyUnroll<T>::value;
  const bool dense = rows == 1 || (dpitch_bytes == width_bytes && spitch_bytes == width_bytes);
  size_t per_row = width_bytes / unit;
  if (dense) {  // one run of rows * width bytes, cut into launches the 32-bit counters cover
    const size_t total = per_row * rows;
    for (size_t at = 0; at < total; at += kCopyMaxUnits) {
      const uint32_t n = static_cast<uint32_t>(std::min<size_t>(kCopyMaxUnits, total - at));
      const unsigned blocks = (n + kPermuteBlock * kCopyUnroll - 1) / (kPermuteBlock * kCopyUnroll);
      hipLaunchKernelGGL((CopyRowsKernel<T, kCopyUnroll, true>), dim3(blocks), dim3(kPermuteBlock), 0, s,
                         static_cast<T *>(dst) + at, size_t(0), static_cast<const T *>(src) + at,
                         size_t(0), n, n, FastDivU32(1));
    }
    return;
  }
  /* pitched: runs of whole rows; a row longer than a launch covers is cut into column runs */
  for (size_t x0 = 0; x0 < per_row; x0 += kCopyMaxUnits) {
    const uint32_t cols = static_cast<uint32_t>(std::min<size_t>(kCopyMaxUnits, per_row - x0));
    const size_t rows_per_launch = std::max<size_t>(1, kCopyMaxUnits / cols);
    for (size_t y0 = 0; y0 < rows; y0 += rows_per_launch) {
      const size_t nrows = std::min(rows_per_launch, rows - y0);
      const uint32_t n = static_cast<uint32_t>(nrows * cols);
      const unsigned blocks = (n + kPermuteBlock * kCopyUnroll - 1) / (kPermuteBlock * kCopyUnroll);
      T *d = reinterpret_cast<T *>(static_cast<char *>(dst) + y0 * dpitch_bytes) + x0;
      const T *f = reinterpret_cast<const T *>(static_cast<const char *>(src) + y0 * spitch_bytes) + x0;
      hipLaunchKernelGGL((CopyRowsKernel<T, kCopyUnroll, false>), dim3(blocks), dim3(kPermuteBlock), 0, s,
                         d, dpitch_bytes / unit, f, spitch_bytes / unit, n, cols, FastDivU32(cols));
    }
  }
}

}  // namespace

namespace mshadow_abi {
/* Copy between two pitched views on the device by a kernel of this library, where everything
   - both addresses, the width and (with more than one row) both pitches - is a multiple of 4
   bytes; false: not covered, the caller uses the runtime's copy. The runtime's own 2-D copy
   reaches 0.73 of the HBM peak on rows of a kilobyte multiple and 0.36 on rows of 127,960
   bytes at a pitch of 128,000; this kernel 0.79-0.81 and 0.71 (8192 rows, MI355X). */
bool CopyRowsOnDevice(void *dst, size_t dpitch_bytes, const void *src, size_t spitch_bytes,
                      size_t width_bytes, size_t rows, hipStream_t s) {
  size_t all = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | width_bytes;
  if (rows > 1) all |= dpitch_bytes | spitch_bytes;
  if (all % 16 == 0) {
    typedef uint32_t Vec __attribute__((ext_vector_type(4)));
    LaunchCopyRows<Vec>(dst, dpitch_bytes, src, spitch_bytes, width_bytes, rows, s);
  } else if (all % 4 == 0 && width_bytes >= 16 && width_bytes < (1ull << 32)) {
    const uint32_t ppr = static_cast<uint32_t>((width_bytes + 15) / 16);
    const size_t rows_per_launch = std::max<size_t>(1, kCopyMaxUnits / ppr);
    for (size_t y0 = 0; y0 < rows; y0 += rows_per_launch) {
      const size_t nrows = std::min(rows_per_launch, rows - y0);
      const uint32_t n = static_cast<uint32_t>(nrows * ppr);
      hipLaunchKernelGGL(CopyRowsAnywhereKernel, dim3((n + kPermuteBlock - 1) / kPermuteBlock),
                         dim3(kPermuteBlock), 0, s, static_cast<char *>(dst) + y0 * dpitch_bytes,
                         dpitch_bytes, static_cast<const char *>(src) + y0 * spitch_bytes, spitch_bytes, n,
                         ppr, static_cast<uint32_t>(width_bytes), FastDivU32(ppr));
    }
  } else if (all % 4 == 0) {
    LaunchCopyRows<uint32_t>(dst, dpitch_bytes, src, spitch_bytes, width_bytes, rows, s);
  } else {
    return false;
  }
  return true;
}
}  // namespace mshadow_abi

/*! \brief whole rows of `packs_per_row` packs one launch of FillKernel covers: it counts packs in
 *  32 bits */
static inline int64_t FillRowsPerLaunch(uint32_t packs_per_row) {
  return static_cast<int64_t>(std::max<uint64_t>(1, ((1ull << 31) - 1) / packs_per_row));
}

/* The runs of rows mshadow_hip_fill_32 launches for a tensor of this shape: first row and row
   count of up to `max_runs` runs into runs[2 * i], runs[2 * i + 1]; returns how many there are.
   No launch, no device: lets the splitting be checked for shapes too large to allocate. */
extern "C" int mshadow_hip_fill_32_runs(int rows, int cols, int wide, int64_t *runs, int max_runs) {
  if (rows <= 0 || cols <= 0) return 0;
  const uint32_t ppr = static_cast<uint32_t>(wide ? cols / 4 : cols);
  if (ppr == 0) return 0;
  const int64_t rows_per_launch = FillRowsPerLaunch(ppr);
  int n = 0;
  for (int64_t row0 = 0; row0 < rows; row0 += rows_per_launch, ++n) {
    if (runs != NULL && n < max_runs) {
      runs[2 * n] = row0;
      runs[2 * n + 1] = std::min<int64_t>(rows_per_launch, rows - row0);
    }
  }
  return n;
}

extern "C" int mshadow_hip_fill_32(void *dst, int dstride, int rows, int cols, uint32_t bits,
                                   void *stream) {
  ABI_REQUIRE(rows >= 0 && cols >= 0, "negative shape");
  if (rows == 0 || cols == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL, "NULL tensor");
  ABI_REQUIRE(dstride >= cols, "pitch smaller than the row");
  const bool wide = cols % 4 == 0 && dstride % 4 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0;
  const uint32_t ppr = static_cast<uint32_t>(wide ? cols / 4 : cols);
  /* the kernel counts packs in 32 bits: a tensor of 2^31 elements or more (it fits this
     device many times over) is filled in runs of whole rows */
  const int64_t rows_per_launch = FillRowsPerLaunch(ppr);
  for (int64_t row0 = 0; row0 < rows; row0 += rows_per_launch) {  // 64-bit: rows may be INT_MAX
    const int64_t nrows = std::min<int64_t>(rows_per_launch, rows - row0);
    uint32_t *first = static_cast<uint32_t *>(dst) + static_cast<size_t>(row0) * dstride;
    uint64_t blocks = (static_cast<uint64_t>(nrows) * ppr + kPermuteBlock - 1) / kPermuteBlock;
    if (blocks > (1u << 20)) blocks = 1u << 20;
    if (wide) {
      hipLaunchKernelGGL(FillKernel<4>, dim3(static_cast<unsigned>(blocks)), dim3(kPermuteBlock), 0,
                         AsStream(stream), first, static_cast<uint32_t>(dstride),
                         static_cast<uint32_t>(nrows), ppr, FastDivU32(ppr), bits);
    } else {
      hipLaunchKernelGGL(FillKernel<1>, dim3(static_cast<unsigned>(blocks)), dim3(kPermuteBlock), 0,
                         AsStream(stream), first, static_cast<uint32_t>(dstride),
                         static_cast<uint32_t>(nrows), ppr, FastDivU32(ppr), bits);
    }
  }
  return AfterLaunch("fill");
}

extern "C" int mshadow_hip_permute_32(void *dst, const void *src, int ndim, const int *shape,
                                      const int *axes, void *stream) {
  ABI_REQUIRE(ndim >= 1 && ndim <= kMaxAxes, "1 to 6 axes");
  ABI_REQUIRE(shape != NULL && axes != NULL, "NULL shape or axes");
  bool seen[kMaxAxes] = {false, false, false, false, false, false};
  uint64_t total = 1;
  for (int i = 0; i < ndim; ++i) {
    ABI_REQUIRE(axes[i] >= 0 && axes[i] < ndim && !seen[axes[i]], "axes is not a permutation");
    ABI_REQUIRE(shape[i] >= 0, "negative shape");
    seen[axes[i]] = true;
    total *= static_cast<uint64_t>(shape[i]);
  }
  if (total == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(total < (1ull << 31), "too many elements");
  ABI_REQUIRE(dst != NULL && src != NULL, "NULL tensor");

  /* reduce: walk the destination axes, drop extents of 1, merge an axis into the previous
     one when the two are neighbours in the source as well */
  uint32_t src_step_of[kMaxAxes];
  {
    uint32_t step = 1;
    for (int k = ndim - 1; k >= 0; --k) {
      src_step_of[k] = step;
      step *= static_cast<uint32_t>(shape[k]);
    }
  }
  uint32_t ext[kMaxAxes], sstep[kMaxAxes];
  int from_axis[kMaxAxes];
  int n = 0;
  for (int i = 0; i < ndim; ++i) {
    const int a = axes[i];
    if (shape[a] == 1) continue;
    if (n > 0 && sstep[n - 1] == src_step_of[a] * static_cast<uint32_t>(shape[a])) {
      ext[n - 1] *= static_cast<uint32_t>(shape[a]);   // (previous, this) is one run of the source
      sstep[n - 1] = src_step_of[a];
      continue;
    }
    ext[n] = static_cast<uint32_t>(shape[a]);
    sstep[n] = src_step_of[a];
    from_axis[n] = a;
    ++n;
  }
  (void)from_axis;
  hipStream_t s = AsStream(stream);
  if (n <= 1) {  // the elements keep their order
    ABI_HIP(hipMemcpyAsync(dst, src, total * sizeof(uint32_t), hipMemcpyDeviceToDevice, s));
    return MSHADOW_HIP_OK;
  }
  uint32_t dstep[kMaxAxes];
  {
    uint32_t step = 1;
    for (int k = n - 1; k >= 0; --k) {
      dstep[k] = step;
      step *= ext[k];
    }
  }
  uint32_t *d = static_cast<uint32_t *>(dst);
  const uint32_t *sp = static_cast<const uint32_t *>(src);
  if (sstep[n - 1] == 1) {
    /* rows of ext[n-1] elements are permuted */
    BatchAxes ba;
    ba.count = n - 1;
    uint32_t rows = 1;
    for (int k = 0; k < n - 1; ++k) {
      ba.extent[k] = FastDivU32(ext[k]);
      ba.src_step[k] = sstep[k];
      ba.dst_step[k] = dstep[k];
      rows *= ext[k];
    }
    const uint32_t cols = ext[n - 1];
    const bool wide = cols % 4 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(src) % 16 == 0;
    const uint32_t ppr = wide ? cols / 4 : cols;
    const uint64_t work = static_cast<uint64_t>(rows) * ppr;
    uint64_t blocks = (work + kPermuteBlock - 1) / kPermuteBlock;
    if (blocks > (1u << 20)) blocks = 1u << 20;
    if (wide) {
      hipLaunchKernelGGL(PermuteRowsKernel<4>, dim3(static_cast<unsigned>(blocks)), dim3(kPermuteBlock),
                         0, s, d, sp, rows, cols, FastDivU32(ppr), ba);
    } else {
      hipLaunchKernelGGL(PermuteRowsKernel<1>, dim3(static_cast<unsigned>(blocks)), dim3(kPermuteBlock),
                         0, s, d, sp, rows, cols, FastDivU32(ppr), ba);
    }
    return AfterLaunch("permute (rows)");
  }
  /* the source's last axis is destination axis b; the destination's last axis is n - 1 */
  int b = -1;
  for (int k = 0; k < n; ++k) {
    if (sstep[k] == 1) b = k;
  }
  ABI_REQUIRE(b >= 0 && b < n - 1, "internal: no unit-stride axis");
  BatchAxes ba;
  ba.count = 0;
  uint64_t batches = 1;
  for (int k = 0; k < n - 1; ++k) {
    if (k == b) continue;
    ba.extent[ba.count] = FastDivU32(ext[k]);
    ba.src_step[ba.count] = sstep[k];
    ba.dst_step[ba.count] = dstep[k];
    ++ba.count;
    batches *= ext[k];
  }
  const uint32_t extent_a = ext[n - 1], extent_l = ext[b];
  const uint32_t ta = (extent_a + kTile - 1) / kTile, tl = (extent_l + kTile - 1) / kTile;
  const uint64_t blocks = batches * ta * tl;
  ABI_REQUIRE(blocks < (1ull << 31), "too many tiles");
  bool wide = extent_a % 4 == 0 && extent_l % 4 == 0 && sstep[n - 1] % 4 == 0 && dstep[b] % 4 == 0 &&
              reinterpret_cast<uintptr_t>(dst) % 16 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0;
  for (int k = 0; k < ba.count; ++k) wide = wide && ba.src_step[k] % 4 == 0 && ba.dst_step[k] % 4 == 0;
  if (wide) {
    hipLaunchKernelGGL(PermuteTileVecKernel, dim3(static_cast<unsigned>(blocks)), dim3(kPermuteBlock),
                       0, s, d, sp, extent_a, extent_l, sstep[n - 1], dstep[b], FastDivU32(ta),
                       FastDivU32(tl), ba);
  } else {
    hipLaunchKernelGGL(PermuteTileKernel, dim3(static_cast<unsigned>(blocks)), dim3(kPermuteBlock), 0,
                       s, d, sp, extent_a, extent_l, sstep[n - 1], dstep[b], FastDivU32(ta),
                       FastDivU32(tl), ba);
  }
  return AfterLaunch("permute (tiles)");
}
