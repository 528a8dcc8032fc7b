/*
 * Pooling forward / backward over the last two dimensions, LDS-tiled.
 *
 * The reference evaluates pool / unpool through its generic map kernel with
 * Plan<PoolingExp>::Eval / Plan<UnPoolingExp>::Eval as the body
 * (mshadow/extension/spatial_pool.h:125-142, spatial_unpool.h:102-125), i.e. ky*kx
 * scattered global loads per output. Here a workgroup stages a band of rows of one
 * (n, c) plane in LDS with coalesced (128-bit where aligned) loads and every window is
 * then read from LDS, so HBM sees each input element once:
 *   pool    reads  planes*h*w*4 B, writes planes*ph*pw*4 B
 *   unpool  reads  planes*(h*w + 2*ph*pw)*4 B, writes planes*h*w*4 B
 * Work inside a band is laid out wave-per-row / lane-per-column, so no integer division
 * is executed per element. Results are bit-identical to the reference: same window
 * clipping, same (y, x) reduction order from the reducer's initial value, `max` / `min`
 * by operator<, and the gradient routed by equality with a separate multiply and add
 * (no fused multiply-add).
 */
#ifndef MSHADOW_AMD_CSRC_POOL_KERNELS_H_
#define MSHADOW_AMD_CSRC_POOL_KERNELS_H_

#include <hip/hip_runtime.h>
#include <mshadow_hip.h>

#include <cfloat>

#include <mshadow/core/fastdiv.h>

#include "stream_access.h"

namespace mshadow_hipk {

const int kPoolBlock = 256;
const int kPoolWaves = kPoolBlock / 64;

template <int REDUCER>
struct PoolOp;
template <>
struct PoolOp<MSHADOW_HIP_SUM> {
  __device__ static float Init() { return 0.0f; }
  __device__ static float Reduce(float d, float s) { return d + s; }
  __device__ static float Grad(float, float) { return 1.0f; }
};
template <>
struct PoolOp<MSHADOW_HIP_MAX> {
  __device__ static float Init() { return -FLT_MAX; }
  __device__ static float Reduce(float d, float s) { return (d < s) ? s : d; }
  __device__ static float Grad(float res, float src) { return res == src ? 1.0f : 0.0f; }
};
template <>
struct PoolOp<MSHADOW_HIP_MIN> {
  __device__ static float Init() { return FLT_MAX; }
  __device__ static float Reduce(float d, float s) { return (s < d) ? s : d; }
  __device__ static float Grad(float res, float src) { return res == src ? 1.0f : 0.0f; }
};

struct PoolGeom {
  int h, w, ph, pw, ky, kx, sy, sx;
  int band;        // output rows (pool) / source rows (unpool) per workgroup
  int bands;       // bands per plane
  int lds_pitch;   // floats per staged row
};

/*! \brief LDS images are shifted by 0..3 floats so that LDS addresses have the same
 *  16-byte phase as the global addresses they mirror: both sides of the staging copy can
 *  then use 128-bit accesses. Callers allocate 4 extra floats per staged array. */
__device__ __forceinline__ int LdsPhase(const float *g) {
  return static_cast<int>((reinterpret_cast<uintptr_t>(g) >> 2) & 3);
}

__device__ __forceinline__ uint32_t IsNegZero(float v) {
  return __float_as_uint(v) == 0x80000000u ? 1u : 0u;
}

/*! \brief copy `nrows` rows of `width` floats (global pitch gpitch) into LDS (pitch
 *  lpitch); `lds` already includes the phase shift of LdsPhase(g). When both pitches equal
 *  the width the band is one contiguous run and moves as 128-bit packs, eight loads in
 *  flight per thread; otherwise one wave takes one row at a time. With WATCH, *neg_zero becomes
 *  non-zero if this thread staged a -0.0f. */
template <bool WATCH = false>
__device__ __forceinline__ void StageRows(float *lds, int lpitch, const float *g, int gpitch,
                                          int nrows, int width, uint32_t *neg_zero = nullptr) {
  uint32_t seen = 0u;
  if (gpitch == width && lpitch == width) {
    const int total = nrows * width;
    const int lead = (4 - LdsPhase(g)) & 3;
    const int head = lead < total ? lead : total;
    if (static_cast<int>(threadIdx.x) < head) {
      const float v = g[threadIdx.x];
      lds[threadIdx.x] = v;
      if (WATCH) seen |= IsNegZero(v);
    }
    const int nvec = (total - head) / 4;
    const float *gv = g + head;
    F4 *lv = reinterpret_cast<F4 *>(lds + head);
    const int kUnroll = 8;
    for (int v0 = threadIdx.x; v0 < nvec; v0 += kPoolBlock * kUnroll) {
      F4 q[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {  // unpredicated: past the end re-reads the last pack
        const int v = v0 + u * kPoolBlock;
        q[u] = StreamLoadF4(gv + 4 * (v < nvec ? v : nvec - 1));
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int v = v0 + u * kPoolBlock;
        if (v < nvec) lv[v] = q[u];
        if (WATCH) seen |= IsNegZero(q[u].x) | IsNegZero(q[u].y) | IsNegZero(q[u].z) | IsNegZero(q[u].w);
      }
    }
    const int tail = head + 4 * nvec + threadIdx.x;
    if (tail < total) {
      const float v = g[tail];
      lds[tail] = v;
      if (WATCH) seen |= IsNegZero(v);
    }
  } else {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int r = wave; r < nrows; r += kPoolWaves) {
      const float *row = g + static_cast<size_t>(r) * gpitch;
      for (int c = lane; c < width; c += 64) {
        const float v = row[c];
        lds[r * lpitch + c] = v;
        if (WATCH) seen |= IsNegZero(v);
      }
    }
  }
  if (WATCH) *neg_zero = seen;
}

/*! \brief max / min of two floats in one instruction. It gives the reference's `(d < s) ? s : d`
 *  / `(s < d) ? s : d` whenever d is not NaN (the running result of a window never is: both forms
 *  pass over a NaN operand) and no -0.0f is about: the comparison keeps the zero it already has,
 *  the instruction takes +0 over -0 (max) or -0 over +0 (min) whichever came first. */
__device__ __forceinline__ float FastMax(float d, float s) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(d), "v"(s));
  return r;
}
__device__ __forceinline__ float FastMin(float d, float s) {
  float r;
  asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(d), "v"(s));
  return r;
}

/*! \brief a whole KY x KX window at `win` (row pitch `pitch`) of a staged band, reduced in the
 *  reference's order; by_comparison = false takes the one-instruction forms (the staged values
 *  then hold no -0.0f) */
template <int REDUCER, int KY, int KX>
__device__ __forceinline__ float ReduceWholeWindow(const float *win, int pitch, bool by_comparison) {
  typedef PoolOp<REDUCER> Op;
  float res = Op::Init();
  if (REDUCER != MSHADOW_HIP_SUM && !by_comparison) {
#pragma unroll
    for (int y = 0; y < KY; ++y) {
#pragma unroll
      for (int x = 0; x < KX; ++x) {
        const float v = win[y * pitch + x];
        res = REDUCER == MSHADOW_HIP_MAX ? FastMax(res, v) : FastMin(res, v);
      }
    }
  } else {
#pragma unroll
    for (int y = 0; y < KY; ++y) {
#pragma unroll
      for (int x = 0; x < KX; ++x) res = Op::Reduce(res, win[y * pitch + x]);
    }
  }
  return res;
}

/*! \brief grid.x = planes * bands. Dynamic LDS: in_rows * lds_pitch + 4 floats, where
 *  in_rows = (band - 1) * sy + ky. KY / KX > 0 fix the window size at compile time
 *  (the loops unroll); 0 means "use g.ky / g.kx". */
template <int REDUCER, int KY, int KX>
__global__ void __launch_bounds__(kPoolBlock)
    PoolKernel(float *dst, int dstride, const float *src, int sstride, PoolGeom g) {
  extern __shared__ float smem[];
  typedef PoolOp<REDUCER> Op;
  const int ky = KY > 0 ? KY : g.ky;
  const int kx = KX > 0 ? KX : g.kx;
  const int plane = blockIdx.x / g.bands;
  const int band = blockIdx.x - plane * g.bands;
  const int py0 = band * g.band;
  const int npy = min(g.band, g.ph - py0);
  const int y0 = py0 * g.sy;
  const int y1 = min(y0 + (npy - 1) * g.sy + ky, g.h);  // one past the last row needed
  const int nrows = max(y1 - y0, 0);
  const float *in = src + (static_cast<size_t>(plane) * g.h + y0) * sstride;
  float *tile = smem + LdsPhase(in);
  /* max and min go by single instructions unless the band holds a -0.0f */
  uint32_t neg_zero = 0u;
  StageRows<REDUCER != MSHADOW_HIP_SUM>(tile, g.lds_pitch, in, sstride, nrows, g.w, &neg_zero);
  const bool by_comparison = __syncthreads_or(static_cast<int>(neg_zero)) != 0;
  float *out = dst + (static_cast<size_t>(plane) * g.ph + py0) * dstride;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int py = wave; py < npy; py += kPoolWaves) {
    const int ys = py * g.sy;  // relative to y0
    const int ye = min(ys + ky, g.h - y0);
    for (int px = lane; px < g.pw; px += 64) {
      const int xs = px * g.sx;
      const int xe = min(xs + kx, g.w);
      float res = Op::Init();
      if (KY > 0 && KX > 0 && ye - ys == KY && xe - xs == KX) {
        res = ReduceWholeWindow<REDUCER, (KY > 0 ? KY : 1), (KX > 0 ? KX : 1)>(
            tile + ys * g.lds_pitch + xs, g.lds_pitch, by_comparison);
      } else {
        for (int y = ys; y < ye; ++y) {
          for (int x = xs; x < xe; ++x) res = Op::Reduce(res, tile[y * g.lds_pitch + x]);
        }
      }
      StreamStore(out + static_cast<size_t>(py) * dstride + px, res);
    }
  }
}

/*! \brief the windows of one staged band when they move by one element (sy == sx == 1, all of
 *  them whole): a thread walks down ONE output column over `run_len` output rows and keeps the
 *  last KY rows of its KX window columns in registers, so that an output costs KX reads of LDS
 *  instead of KY * KX. The `nruns` runs of the band times its pw columns are dealt over the
 *  threads; lanes of a wave sit in neighbouring columns. The order of the reduction inside a
 *  window is the reference's (rows outermost). */
template <int REDUCER, int KY, int KX>
__device__ __forceinline__ void ColumnsS1Band(float *out, int dstride, const float *tile, int pitch, int npy,
                                              int pw, int nruns, int run_len, mshadow::FastDivU32 div_pw,
                                              bool by_comparison) {
  typedef PoolOp<REDUCER> Op;
  const uint32_t items = static_cast<uint32_t>(nruns) * pw;
  for (uint32_t it = threadIdx.x; it < items; it += kPoolBlock) {
    const uint32_t run = div_pw.Div(it);
    const int px = static_cast<int>(it - run * pw);
    const int r0 = static_cast<int>(run) * run_len;
    const int nr = min(run_len, npy - r0);
    if (nr <= 0) continue;
    const float *col = tile + r0 * pitch + px;
    float *o = out + static_cast<size_t>(r0) * dstride + px;
    float ring[KY][KX];  // input row t of the run sits in slot t % KY
#pragma unroll
    for (int y = 0; y < KY - 1; ++y) {
#pragma unroll
      for (int x = 0; x < KX; ++x) ring[y][x] = col[y * pitch + x];
    }
    for (int r = 0; r < nr; r += KY) {
#pragma unroll
      for (int j = 0; j < KY; ++j) {
        if (r + j < nr) {
#pragma unroll
          for (int x = 0; x < KX; ++x) ring[(j + KY - 1) % KY][x] = col[(r + j + KY - 1) * pitch + x];
          float res = Op::Init();
          if (REDUCER != MSHADOW_HIP_SUM && !by_comparison) {
#pragma unroll
            for (int y = 0; y < KY; ++y) {
#pragma unroll
              for (int x = 0; x < KX; ++x) {
                const float v = ring[(j + y) % KY][x];
                res = REDUCER == MSHADOW_HIP_MAX ? FastMax(res, v) : FastMin(res, v);
              }
            }
          } else {
#pragma unroll
            for (int y = 0; y < KY; ++y) {
#pragma unroll
              for (int x = 0; x < KX; ++x) res = Op::Reduce(res, ring[(j + y) % KY][x]);
            }
          }
          /* an ordinary store: output rows are as many bytes as input rows here and seldom end on
             a cache line, and the lines two rows share leave L2 whole this way ((128,64,112,112)
             3x3: 151 us against 162 us with streaming stores) */
          o[static_cast<size_t>(r + j) * dstride] = res;
        }
      }
    }
  }
}

/*! \brief stride-1 pooling, one band of one plane per workgroup, staged as in PoolKernel.
 *  grid.x = planes * bands. */
template <int REDUCER, int KY, int KX>
__global__ void __launch_bounds__(kPoolBlock)
    PoolColumnsS1Kernel(float *dst, int dstride, const float *src, int sstride, PoolGeom g, int nruns,
                        int run_len, mshadow::FastDivU32 div_pw) {
  extern __shared__ float smem[];
  const int plane = blockIdx.x / g.bands;
  const int band = blockIdx.x - plane * g.bands;
  const int py0 = band * g.band;
  const int npy = min(g.band, g.ph - py0);
  const int nrows = npy + KY - 1;
  const float *in = src + (static_cast<size_t>(plane) * g.h + py0) * sstride;
  float *tile = smem + LdsPhase(in);
  uint32_t neg_zero = 0u;
  StageRows<REDUCER != MSHADOW_HIP_SUM>(tile, g.lds_pitch, in, sstride, nrows, g.w, &neg_zero);
  const bool by_comparison = __syncthreads_or(static_cast<int>(neg_zero)) != 0;
  float *out = dst + (static_cast<size_t>(plane) * g.ph + py0) * dstride;
  ColumnsS1Band<REDUCER, KY, KX>(out, dstride, tile, g.lds_pitch, npy, g.pw, nruns, run_len, div_pw,
                                 by_comparison);
}

/*! \brief The same for small planes: a workgroup takes `per_block` whole consecutive planes (they
 *  are consecutive rows of the tensor's 2-D view, so their rows stage as one band) and computes
 *  all their windows; with one small plane per workgroup the launch of the workgroups is what
 *  takes the time ((256,256,13,13), 3x3 stride 2: 91 us for 54 MB). grid.x = ceil(planes /
 *  per_block); dynamic LDS: per_block * h * lds_pitch + 4 floats. */
template <int REDUCER, int KY, int KX>
__global__ void __launch_bounds__(kPoolBlock)
    PoolPlanesKernel(float *dst, int dstride, const float *src, int sstride, PoolGeom g, int planes,
                     int per_block, mshadow::FastDivU32 div_ph) {
  extern __shared__ float smem[];
  typedef PoolOp<REDUCER> Op;
  const int ky = KY > 0 ? KY : g.ky;
  const int kx = KX > 0 ? KX : g.kx;
  const int plane0 = blockIdx.x * per_block;
  const int np = min(per_block, planes - plane0);
  const float *in = src + static_cast<size_t>(plane0) * g.h * sstride;
  float *tile = smem + LdsPhase(in);
  uint32_t neg_zero = 0u;
  StageRows<REDUCER != MSHADOW_HIP_SUM>(tile, g.lds_pitch, in, sstride, np * g.h, g.w, &neg_zero);
  const bool by_comparison = __syncthreads_or(static_cast<int>(neg_zero)) != 0;
  float *out = dst + static_cast<size_t>(plane0) * g.ph * dstride;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  /* a wave takes `rpw` output rows at a time, pw lanes each (64 / pw of them, at least one) */
  const int rpw = g.pw >= 64 ? 1 : 64 / g.pw;
  const int sub = rpw == 1 ? 0 : lane / g.pw;
  const int px0 = rpw == 1 ? lane : lane - sub * g.pw;
  const int rows_out = np * g.ph;
  for (int r0 = wave * rpw; r0 < rows_out; r0 += kPoolWaves * rpw) {
    const int r = r0 + sub;
    if (sub >= rpw || r >= rows_out) continue;
    const int p = static_cast<int>(div_ph.Div(static_cast<uint32_t>(r)));
    const int py = r - p * g.ph;
    const int ys = p * g.h + py * g.sy;
    const int ye = min(ys + ky, (p + 1) * g.h);
    for (int px = px0; px < g.pw; px += (rpw == 1 ? 64 : g.pw)) {
      const int xs = px * g.sx;
      const int xe = min(xs + kx, g.w);
      float res = Op::Init();
      if (KY > 0 && KX > 0 && ye - ys == KY && xe - xs == KX) {
        res = ReduceWholeWindow<REDUCER, (KY > 0 ? KY : 1), (KX > 0 ? KX : 1)>(
            tile + ys * g.lds_pitch + xs, g.lds_pitch, by_comparison);
      } else {
        for (int y = ys; y < ye; ++y) {
          for (int x = xs; x < xe; ++x) res = Op::Reduce(res, tile[y * g.lds_pitch + x]);
        }
      }
      StreamStore(out + static_cast<size_t>(r) * dstride + px, res);
    }
  }
}

/*! \brief no staging: used when even one band of rows does not fit in LDS */
template <int REDUCER>
__global__ void __launch_bounds__(kPoolBlock)
    PoolDirectKernel(float *dst, int dstride, const float *src, int sstride, PoolGeom g,
                     unsigned total) {
  typedef PoolOp<REDUCER> Op;
  for (unsigned o = blockIdx.x * kPoolBlock + threadIdx.x; o < total; o += gridDim.x * kPoolBlock) {
    const unsigned i = o / g.pw;
    const int px = o - i * g.pw;
    const int py = i % g.ph;
    const int plane = i / g.ph;
    const int ys = py * g.sy, ye = min(ys + g.ky, g.h);
    const int xs = px * g.sx, xe = min(xs + g.kx, g.w);
    float res = Op::Init();
    for (int y = ys; y < ye; ++y) {
      const float *row = src + (static_cast<size_t>(plane) * g.h + y) * sstride;
      for (int x = xs; x < xe; ++x) res = Op::Reduce(res, row[x]);
    }
    dst[static_cast<size_t>(i) * dstride + px] = res;
  }
}

/*! \brief grid.x = planes * bands over SOURCE rows. Dynamic LDS: two arrays (pooled,
 *  grad) of prow_max * lds_pitch + 4 floats, prow_max = (band + ky - 2) / sy + 2.
 *  KY, KX, SY, SX > 0 fix the window and stride at compile time: the number of windows
 *  that can cover a pixel, ceil(K / S) per direction, is then a constant, the loops unroll
 *  and the range divisions become shifts. 0 means "use the run-time value". A candidate
 *  window that does not exist is skipped with a select, which leaves `val` untouched
 *  exactly like the reference's loop bounds do. */
template <int REDUCER, int KY, int KX, int SY, int SX>
__global__ void __launch_bounds__(kPoolBlock)
    UnpoolKernel(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                 int pstride, const float *grad, int gstride, PoolGeom g, int prow_max) {
  extern __shared__ float smem[];
  typedef PoolOp<REDUCER> Op;
  const bool kFixed = KY > 0 && KX > 0 && SY > 0 && SX > 0;
  if (kFixed) {
    g.ky = KY; g.kx = KX; g.sy = SY; g.sx = SX;
  }
  const int plane = blockIdx.x / g.bands;
  const int band = blockIdx.x - plane * g.bands;
  const int y0 = band * g.band;
  const int ny = min(g.band, g.h - y0);
  const int ylast = y0 + ny - 1;
  /* pooled rows touched by source rows y0..ylast */
  const int p0 = y0 < g.ky ? 0 : (y0 - g.ky + g.sy) / g.sy;
  const int p1 = min((ylast + g.sy) / g.sy, g.ph);
  const int np = max(p1 - p0, 0);
  const float *pin = pooled + (static_cast<size_t>(plane) * g.ph + p0) * pstride;
  const float *gin = grad + (static_cast<size_t>(plane) * g.ph + p0) * gstride;
  float *sp = smem + LdsPhase(pin);
  float *sg = smem + prow_max * g.lds_pitch + 4 + LdsPhase(gin);
  StageRows(sp, g.lds_pitch, pin, pstride, np, g.pw);
  StageRows(sg, g.lds_pitch, gin, gstride, np, g.pw);
  const float *in = src + (static_cast<size_t>(plane) * g.h + y0) * sstride;
  float *out = dst + (static_cast<size_t>(plane) * g.h + y0) * dstride;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  /* each lane fetches its source pixel of kRowsAhead rows before using any of them */
  const int kRowsAhead = 4;
  const int kCandY = kFixed ? (KY + SY - 1) / (SY > 0 ? SY : 1) : 1;
  const int kCandX = kFixed ? (KX + SX - 1) / (SX > 0 ? SX : 1) : 1;
  __syncthreads();
  for (int yr0 = wave; yr0 < ny; yr0 += kPoolWaves * kRowsAhead) {
    for (int x = lane; x < g.w; x += 64) {
      float vs[kRowsAhead];
#pragma unroll
      for (int u = 0; u < kRowsAhead; ++u) {
        const int yr = yr0 + u * kPoolWaves;
        vs[u] = (yr < ny) ? StreamLoad(in + static_cast<size_t>(yr) * sstride + x) : 0.0f;
      }
      const int px_min = x < g.kx ? 0 : (x - g.kx + g.sx) / g.sx;
      const int px_max = min((x + g.sx) / g.sx, g.pw);
#pragma unroll
      for (int u = 0; u < kRowsAhead; ++u) {
        const int yr = yr0 + u * kPoolWaves;
        if (yr < ny) {
          const int y = y0 + yr;
          const int py_min = y < g.ky ? 0 : (y - g.ky + g.sy) / g.sy;
          const int py_max = min((y + g.sy) / g.sy, g.ph);
          float val = 0.0f;
          if (kFixed) {
#pragma unroll
            for (int iy = 0; iy < kCandY; ++iy) {
              const int py = py_min + iy;
#pragma unroll
              for (int ix = 0; ix < kCandX; ++ix) {
                const int px = px_min + ix;
                const bool live = py < py_max && px < px_max;
                /* clamp the LDS index of a missing candidate into the staged area */
                const int li = live ? (py - p0) * g.lds_pitch + px : 0;
                const float t = val + Op::Grad(vs[u], sp[li]) * sg[li];
                val = live ? t : val;
              }
            }
          } else {
            for (int py = py_min; py < py_max; ++py) {
              for (int px = px_min; px < px_max; ++px) {
                const int li = (py - p0) * g.lds_pitch + px;
                val = val + Op::Grad(vs[u], sp[li]) * sg[li];
              }
            }
          }
          StreamStore(out + static_cast<size_t>(yr) * dstride + x, val);
        }
      }
    }
  }
}

/*! \brief unpool with no staging, any window and stride, rows of four pixels or more: a thread
 *  takes four neighbouring source pixels (one 16-byte access each way, at any alignment; the
 *  last pack of a row moved back to end with the row) and, pixel by pixel, the windows that
 *  cover it in the reference's order (py, then px ascending;
 *  mshadow/extension/spatial_unpool.h:102-125), their pooled values and gradients by
 *  element-sized loads that neighbouring pixels and lanes share cache lines for. */
template <int REDUCER>
__global__ void __launch_bounds__(kPoolBlock)
    UnpoolGatherKernel(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                       int pstride, const float *grad, int gstride, PoolGeom g,
                       mshadow::FastDivU32 div_sy, mshadow::FastDivU32 div_sx,
                       mshadow::FastDivU32 div_wpk, mshadow::FastDivU32 div_h, uint32_t total_packs) {
  typedef PoolOp<REDUCER> Op;
  const uint32_t pk = blockIdx.x * kPoolBlock + threadIdx.x;
  if (pk >= total_packs) return;
  const uint32_t r = div_wpk.Div(pk);                // plane * h + y
  const int x0 = min(static_cast<int>(pk - r * div_wpk.div) * 4, g.w - 4);
  const uint32_t plane = div_h.Div(r);
  const int y = static_cast<int>(r - plane * g.h);
  const F4 vs = StreamLoadF4Anywhere(src + static_cast<size_t>(r) * sstride + x0);
  const int py_min = y < g.ky ? 0 : static_cast<int>(div_sy.Div(y - g.ky + g.sy));
  const int py_max = min(static_cast<int>(div_sy.Div(y + g.sy)), g.ph);
  const float *prow = pooled + static_cast<size_t>(plane) * g.ph * pstride;
  const float *grow = grad + static_cast<size_t>(plane) * g.ph * gstride;
  F4 out;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int x = x0 + e;
    const int px_min = x < g.kx ? 0 : static_cast<int>(div_sx.Div(x - g.kx + g.sx));
    const int px_max = min(static_cast<int>(div_sx.Div(x + g.sx)), g.pw);
    float val = 0.0f;
    for (int py = py_min; py < py_max; ++py) {
      for (int px = px_min; px < px_max; ++px) {
        val = val + Op::Grad(vs[e], prow[static_cast<size_t>(py) * pstride + px]) *
                        grow[static_cast<size_t>(py) * gstride + px];
      }
    }
    out[e] = val;
  }
  StreamStoreF4Anywhere(dst + static_cast<size_t>(r) * dstride + x0, out);
}

/*! \brief two floats fetched as one 8-byte access at any 4-byte boundary */
typedef F2 F2Loose __attribute__((aligned(4)));

/*! \brief unpool for 2 x 2 windows with stride 2 - windows that do not overlap, so a source
 *  pixel has at most one - with no staging: a thread takes four neighbouring source pixels of
 *  one row (one 16-byte access each way, any alignment), which lie under two neighbouring windows of one pooled row, and fetches the
 *  pooled values and gradients of those two as one 8-byte access each. The single term is
 *  added to zero as the reference's loop does (mshadow/extension/spatial_unpool.h:102-125). */
template <int REDUCER>
__global__ void __launch_bounds__(kPoolBlock)
    Unpool2x2s2Kernel(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                      int pstride, const float *grad, int gstride, PoolGeom g,
                      mshadow::FastDivU32 div_wpk, mshadow::FastDivU32 div_h, uint32_t total_packs) {
  typedef PoolOp<REDUCER> Op;
  const uint32_t pk = blockIdx.x * kPoolBlock + threadIdx.x;
  if (pk >= total_packs) return;
  const uint32_t r = div_wpk.Div(pk);                // plane * h + y
  int x0 = static_cast<int>(pk - r * div_wpk.div) * 4;
  /* the last pack of a row of even width is moved back to end with the row (it still starts a
     window); of an odd width it is partial */
  if (x0 + 4 > g.w && (g.w & 1) == 0) x0 = g.w - 4;
  const uint32_t plane = div_h.Div(r);
  const int y = static_cast<int>(r - plane * g.h);
  const int py = y >> 1, px = x0 >> 1;
  const float *in = src + static_cast<size_t>(r) * sstride + x0;
  float *out = dst + static_cast<size_t>(r) * dstride + x0;
  const int live = min(4, g.w - x0);                 // 4, or 3 when the width is odd
  float vs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (live == 4) {
    const F4 q = StreamLoadF4Anywhere(in);
    vs[0] = q.x; vs[1] = q.y; vs[2] = q.z; vs[3] = q.w;
  } else {
    for (int e = 0; e < live; ++e) vs[e] = in[e];
  }
  float pv[2] = {0.0f, 0.0f}, gv[2] = {0.0f, 0.0f};
  const bool row_ok = py < g.ph;
  if (row_ok) {
    const float *prow = pooled + (static_cast<size_t>(plane) * g.ph + py) * pstride + px;
    const float *grow = grad + (static_cast<size_t>(plane) * g.ph + py) * gstride + px;
    if (px + 2 <= g.pw) {
      const F2 a = *reinterpret_cast<const F2Loose *>(prow);
      const F2 b = *reinterpret_cast<const F2Loose *>(grow);
      pv[0] = a.x; pv[1] = a.y; gv[0] = b.x; gv[1] = b.y;
    } else if (px < g.pw) {
      pv[0] = prow[0];
      gv[0] = grow[0];
    }
  }
  float o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const bool has = row_ok && px + (e >> 1) < g.pw;
    const float t = 0.0f + Op::Grad(vs[e], pv[e >> 1]) * gv[e >> 1];
    o[e] = has ? t : 0.0f;
  }
  if (live == 4) {
    F4 q;
    q.x = o[0]; q.y = o[1]; q.z = o[2]; q.w = o[3];
    StreamStoreF4Anywhere(out, q);
  } else {
    for (int e = 0; e < live; ++e) out[e] = o[e];
  }
}

/*! \brief unpool for small planes: a workgroup takes `per_block` whole consecutive planes, stages
 *  their pooled values and gradients (per_block * ph rows each) and computes every source pixel
 *  of those planes; a wave takes 64 / w source rows at a time when rows are short. Terms in
 *  the reference's order (py, then px ascending; mshadow/extension/spatial_unpool.h:102-125), a
 *  multiply and an add each. grid.x = ceil(planes / per_block); dynamic LDS: two arrays of
 *  per_block * ph * lds_pitch + 4 floats. */
template <int REDUCER, int KY, int KX, int SY, int SX>
__global__ void __launch_bounds__(kPoolBlock)
    UnpoolPlanesKernel(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                       int pstride, const float *grad, int gstride, PoolGeom g, int planes,
                       int per_block, mshadow::FastDivU32 div_h) {
  extern __shared__ float smem[];
  typedef PoolOp<REDUCER> Op;
  const bool kFixed = KY > 0 && KX > 0 && SY > 0 && SX > 0;
  if (kFixed) {   // window and stride known to the compiler: the range divisions become shifts
    g.ky = KY; g.kx = KX; g.sy = SY; g.sx = SX;
  }
  const int kCandY = kFixed ? (KY + SY - 1) / (SY > 0 ? SY : 1) : 1;
  const int kCandX = kFixed ? (KX + SX - 1) / (SX > 0 ? SX : 1) : 1;
  const int plane0 = blockIdx.x * per_block;
  const int np = min(per_block, planes - plane0);
  const float *pin = pooled + static_cast<size_t>(plane0) * g.ph * pstride;
  const float *gin = grad + static_cast<size_t>(plane0) * g.ph * gstride;
  float *sp = smem + LdsPhase(pin);
  float *sg = smem + per_block * g.ph * g.lds_pitch + 4 + LdsPhase(gin);
  StageRows(sp, g.lds_pitch, pin, pstride, np * g.ph, g.pw);
  StageRows(sg, g.lds_pitch, gin, gstride, np * g.ph, g.pw);
  __syncthreads();
  const float *in = src + static_cast<size_t>(plane0) * g.h * sstride;
  float *out = dst + static_cast<size_t>(plane0) * g.h * dstride;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int rpw = g.w >= 64 ? 1 : 64 / g.w;
  const int sub = rpw == 1 ? 0 : lane / g.w;
  const int x0 = rpw == 1 ? lane : lane - sub * g.w;
  const int rows = np * g.h;
  for (int r0 = wave * rpw; r0 < rows; r0 += kPoolWaves * rpw) {
    const int r = r0 + sub;
    if (sub >= rpw || r >= rows) continue;
    const int p = static_cast<int>(div_h.Div(static_cast<uint32_t>(r)));
    const int y = r - p * g.h;
    const int py_min = y < g.ky ? 0 : (y - g.ky + g.sy) / g.sy;
    const int py_max = min((y + g.sy) / g.sy, g.ph);
    for (int x = x0; x < g.w; x += (rpw == 1 ? 64 : g.w)) {
      const float vs = StreamLoad(in + static_cast<size_t>(r) * sstride + x);
      const int px_min = x < g.kx ? 0 : (x - g.kx + g.sx) / g.sx;
      const int px_max = min((x + g.sx) / g.sx, g.pw);
      float val = 0.0f;
      if (kFixed) {
#pragma unroll
        for (int iy = 0; iy < kCandY; ++iy) {
          const int py = py_min + iy;
#pragma unroll
          for (int ix = 0; ix < kCandX; ++ix) {
            const int px = px_min + ix;
            const bool live = py < py_max && px < px_max;
            const int li = live ? (p * g.ph + py) * g.lds_pitch + px : 0;
            const float t = val + Op::Grad(vs, sp[li]) * sg[li];
            val = live ? t : val;
          }
        }
      } else {
        for (int py = py_min; py < py_max; ++py) {
          for (int px = px_min; px < px_max; ++px) {
            const int li = (p * g.ph + py) * g.lds_pitch + px;
            val = val + Op::Grad(vs, sp[li]) * sg[li];
          }
        }
      }
      StreamStore(out + static_cast<size_t>(r) * dstride + x, val);
    }
  }
}

/*! \brief unpool for a window and stride fixed at compile time, one thread per SY x SX
 *  block of source pixels aligned to the stride. The windows that can cover a pixel of the
 *  block at (a, b) are (a - jy, b - jx), jy < ceil(KY / SY), jx < ceil(KX / SX): the
 *  pooled value and the gradient of each are read from LDS once per block (not once per
 *  pixel), and which of them cover which pixel of the block - jy * SY + dy < KY - is known
 *  to the compiler, so only existing terms are evaluated, in the reference's py, px order.
 *  VEC: rows are made of whole blocks and are aligned, a block row moves as one access.
 *  Same grid and LDS layout as UnpoolKernel; bands start at multiples of SY. */
template <int REDUCER, int KY, int KX, int SY, int SX, bool VEC>
__global__ void __launch_bounds__(kPoolBlock)
    UnpoolBlockKernel(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                      int pstride, const float *grad, int gstride, PoolGeom g, int prow_max,
                      mshadow::FastDivU32 div_bw) {
  extern __shared__ float smem[];
  typedef PoolOp<REDUCER> Op;
  const int JY = (KY + SY - 1) / SY, JX = (KX + SX - 1) / SX;
  const int plane = blockIdx.x / g.bands;
  const int band = blockIdx.x - plane * g.bands;
  const int y0 = band * g.band;
  const int ny = min(g.band, g.h - y0);
  const int ylast = y0 + ny - 1;
  const int p0 = y0 < KY ? 0 : (y0 - KY + SY) / SY;
  const int p1 = min((ylast + SY) / SY, g.ph);
  const int np = max(p1 - p0, 0);
  const float *pin = pooled + (static_cast<size_t>(plane) * g.ph + p0) * pstride;
  const float *gin = grad + (static_cast<size_t>(plane) * g.ph + p0) * gstride;
  float *sp = smem + LdsPhase(pin);
  float *sg = smem + prow_max * g.lds_pitch + 4 + LdsPhase(gin);
  StageRows(sp, g.lds_pitch, pin, pstride, np, g.pw);
  StageRows(sg, g.lds_pitch, gin, gstride, np, g.pw);
  const float *in = src + (static_cast<size_t>(plane) * g.h + y0) * sstride;
  float *out = dst + (static_cast<size_t>(plane) * g.h + y0) * dstride;
  const int bw = (g.w + SX - 1) / SX;
  const int a0 = y0 / SY;
  const unsigned nblk = static_cast<unsigned>((ny + SY - 1) / SY) * bw;
  const int kAhead = 4;  // blocks per thread whose loads are issued before any is used
  __syncthreads();
  for (unsigned t0 = threadIdx.x; t0 < nblk; t0 += kPoolBlock * kAhead) {
    float vs[kAhead][SY][SX];
    int ar[kAhead], b[kAhead];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      /* past the end: re-read the last block (unpredicated loads), nothing is stored */
      const unsigned t = min(t0 + u * kPoolBlock, nblk - 1);
      ar[u] = static_cast<int>(div_bw.Div(t));
      b[u] = static_cast<int>(t) - ar[u] * bw;
#pragma unroll
      for (int dy = 0; dy < SY; ++dy) {
        const int yr = min(ar[u] * SY + dy, ny - 1);
        const float *row = in + static_cast<size_t>(yr) * sstride + b[u] * SX;
        if (VEC) {
          StreamLoadN<SX>(vs[u][dy], row);
        } else {
#pragma unroll
          for (int dx = 0; dx < SX; ++dx) vs[u][dy][dx] = StreamLoad(row + min(dx, g.w - 1 - b[u] * SX));
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      if (t0 + u * kPoolBlock >= nblk) break;
      float pv[JY][JX], gv[JY][JX];
      bool ok[JY][JX];
#pragma unroll
      for (int jy = 0; jy < JY; ++jy) {
#pragma unroll
        for (int jx = 0; jx < JX; ++jx) {
          const int py = a0 + ar[u] - jy, px = b[u] - jx;
          ok[jy][jx] = py >= 0 && py < g.ph && px >= 0 && px < g.pw;
          /* a window that does not exist reads slot 0 and is skipped by the select below */
          const int li = ok[jy][jx] ? (py - p0) * g.lds_pitch + px : 0;
          pv[jy][jx] = sp[li];
          gv[jy][jx] = sg[li];
        }
      }
#pragma unroll
      for (int dy = 0; dy < SY; ++dy) {
        const int yr = ar[u] * SY + dy;
        float val[SX];
#pragma unroll
        for (int dx = 0; dx < SX; ++dx) {
          val[dx] = 0.0f;
#pragma unroll
          for (int jy = JY - 1; jy >= 0; --jy) {      // py ascending
            if (jy * SY + dy >= KY) continue;         // this window row does not reach the pixel
#pragma unroll
            for (int jx = JX - 1; jx >= 0; --jx) {    // px ascending
              if (jx * SX + dx >= KX) continue;
              const float t = val[dx] + Op::Grad(vs[u][dy][dx], pv[jy][jx]) * gv[jy][jx];
              val[dx] = ok[jy][jx] ? t : val[dx];
            }
          }
        }
        if (yr < ny) {
          float *orow = out + static_cast<size_t>(yr) * dstride + b[u] * SX;
          if (VEC) {
            StreamStoreN<SX>(orow, val);
          } else {
#pragma unroll
            for (int dx = 0; dx < SX; ++dx) {
              if (b[u] * SX + dx < g.w) StreamStore(orow + dx, val[dx]);
            }
          }
        }
      }
    }
  }
}

/*! \brief geometry of UnpoolRows3x3s2Kernel: the pairs of source rows (2a, 2a + 1) of all
 *  planes are numbered plane * (h / 2) + a; a wave takes `rows_per_wave` consecutive ones,
 *  `groups` = w / 4 lanes each */
struct UnpoolRowsGeom {
  uint32_t total_rows, groups, rows_per_wave, half_h;
  size_t pooled_floats, grad_floats;   // extent of the two pooled-size arrays, last row unpadded
  size_t src_floats;                   // extent of the source, last row unpadded
  mshadow::FastDivU32 div_groups, div_half_h;
};

__device__ __forceinline__ F4 LoadPackFree(const float *base, const float *p, const float *end, bool ok);

/*! \brief unpool for a 3 x 3 window with stride 2 on rows of up to 256 pixels, with no staging:
 *  a thread owns two adjacent 2 x 2 blocks of source pixels - four pixels of row 2a and the four
 *  below them. RAGGED = false: h even, w a multiple of 4, rows of whole aligned packs. RAGGED =
 *  true: any h and w at any alignment - the last pair of rows of an odd height has no lower row,
 *  the last pack of a row that is not whole packs is fetched whole (what lies behind the row is
 *  the next row's and is not stored) and stored element by element; every load of this form sits
 *  outside any branch and is issued before the first value is used, so a thread waits for memory
 *  once ((64,96,55,55): 52 -> 48 us; with loads inside the branches of the two cases the
 *  compiler waits for all loads under way at each). What this form still pays against the other
 *  (33 us on 56 x 56) are 16-byte accesses at 4-byte borders. The windows that can cover them
 *  are rows a - 1 and a of the pooled grid, columns 2t - 1, 2t, 2t + 1: the thread fetches
 *  columns 2t and 2t + 1 of both rows (pooled value and gradient) and takes column 2t - 1
 *  from the neighbouring lane, which fetched it as its own 2t' + 1 (a wave takes whole rows).
 *  Source and result move as 128-bit accesses; nothing is staged and there is no barrier.
 *  Terms in the reference's order (py, then px ascending; mshadow/extension/
 *  spatial_unpool.h:102-125), a multiply and an add each. */
template <int REDUCER, bool RAGGED>
__global__ void __launch_bounds__(kPoolBlock)
    UnpoolRows3x3s2Kernel(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                          int pstride, const float *grad, int gstride, PoolGeom g, UnpoolRowsGeom rg) {
  typedef PoolOp<REDUCER> Op;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = blockIdx.x * (kPoolBlock / 64) + (threadIdx.x >> 6);
  const uint32_t row_in_wave = rg.div_groups.Div(lane);
  const uint32_t t = lane - row_in_wave * rg.groups;
  const uint32_t brow = wave * rg.rows_per_wave + row_in_wave;
  const bool live = row_in_wave < rg.rows_per_wave && brow < rg.total_rows;
  const uint32_t browc = live ? brow : rg.total_rows - 1u;
  const uint32_t plane = rg.div_half_h.Div(browc);
  const int a = static_cast<int>(browc - plane * rg.half_h);
  const float *in = src + (static_cast<size_t>(plane) * g.h + 2 * a) * sstride + 4u * t;
  const int live_px = RAGGED ? min(4, g.w - static_cast<int>(4u * t)) : 4;
  const bool has_bottom = !RAGGED || 2 * a + 1 < g.h;
  F4 top, bottom;
  if (!RAGGED) {
    top = StreamLoadF4(in), bottom = StreamLoadF4(in + sstride);
  } else {
    const float *send = src + rg.src_floats;
    top = LoadPackFree(src, in, send, true);
    bottom = LoadPackFree(src, in + sstride, send, has_bottom);
  }
  /* [jy][c]: pooled row a - jy, column 2t - 1 + c */
  float pv[2][3], gv[2][3];
  bool ok[2][3];
  if (RAGGED) {
    /* both pooled rows of both arrays requested at once: columns 2t and 2t + 1 as one 8-byte
       access; only the last float of an array has nothing behind it, and is fetched as the
       second of the pair before it */
#pragma unroll
    for (int jy = 0; jy < 2; ++jy) {
      const int py = a - jy;
      const bool row_ok = py >= 0 && py < g.ph;
      const size_t prow = static_cast<size_t>(plane) * g.ph + (row_ok ? py : 0);
      const int px = static_cast<int>(2u * t);
      const int pxc = px < g.pw ? px : 0;
      const size_t poff = prow * pstride + pxc, goff = prow * gstride + pxc;
      const bool ptail = poff + 2 > rg.pooled_floats, gtail = goff + 2 > rg.grad_floats;
      const F2 pp = *reinterpret_cast<const F2Loose *>(pooled + poff - (ptail ? 1 : 0));
      const F2 gg = *reinterpret_cast<const F2Loose *>(grad + goff - (gtail ? 1 : 0));
      pv[jy][1] = ptail ? pp.y : pp.x, pv[jy][2] = pp.y;
      gv[jy][1] = gtail ? gg.y : gg.x, gv[jy][2] = gg.y;
    }
  }
#pragma unroll
  for (int jy = 0; jy < 2; ++jy) {
    const int py = a - jy;
    const bool row_ok = py >= 0 && py < g.ph;
    const size_t prow = static_cast<size_t>(plane) * g.ph + (row_ok ? py : 0);
    /* columns 2t and 2t + 1 as one 8-byte access per array; a window that does not exist reads
       an existing float (the next row's first at most) and is skipped below. Only the last
       floats of the two arrays have nothing behind them: there the columns come one by one */
    const int px = static_cast<int>(2u * t);
    const int pxc = px < g.pw ? px : 0;
    const size_t poff = prow * pstride + pxc, goff = prow * gstride + pxc;
    /* pooled row a - 1 is row a' of the pair above, which the lanes `groups` below hold when
       that pair is in this wave and plane */
    const bool from_above = !RAGGED && jy == 1 && row_in_wave > 0u && a > 0 && live;
    if (RAGGED) {
      /* fetched above */
    } else if (from_above) {
      pv[jy][1] = pv[jy][2] = gv[jy][1] = gv[jy][2] = 0.0f;
    } else if (poff + 2 <= rg.pooled_floats && goff + 2 <= rg.grad_floats) {
      const F2 pp = *reinterpret_cast<const F2Loose *>(pooled + poff);
      const F2 gg = *reinterpret_cast<const F2Loose *>(grad + goff);
      pv[jy][1] = pp.x, pv[jy][2] = pp.y;
      gv[jy][1] = gg.x, gv[jy][2] = gg.y;
    } else {
      pv[jy][1] = pv[jy][2] = pooled[poff];
      gv[jy][1] = gv[jy][2] = grad[goff];
    }
    if (jy == 1 && !RAGGED) {
      const int from = from_above ? static_cast<int>(lane - rg.groups) : static_cast<int>(lane);
      const float p1 = __shfl(pv[0][1], from), p2 = __shfl(pv[0][2], from);
      const float g1 = __shfl(gv[0][1], from), g2 = __shfl(gv[0][2], from);
      if (from_above) pv[1][1] = p1, pv[1][2] = p2, gv[1][1] = g1, gv[1][2] = g2;
    }
    ok[jy][1] = row_ok && px < g.pw;
    ok[jy][2] = row_ok && px + 1 < g.pw;
    /* column 2t - 1 is the neighbour's 2t' + 1 (every lane takes part in the exchange) */
    pv[jy][0] = __uint_as_float(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(
        0, static_cast<int>(__float_as_uint(pv[jy][2])), 0x138, 0xf, 0xf, false)));
    gv[jy][0] = __uint_as_float(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(
        0, static_cast<int>(__float_as_uint(gv[jy][2])), 0x138, 0xf, 0xf, false)));
    ok[jy][0] = row_ok && t > 0u && static_cast<int>(2u * t) - 1 < g.pw;
  }
  if (!live) return;
  const float vtop[4] = {top.x, top.y, top.z, top.w};
  const float vbot[4] = {bottom.x, bottom.y, bottom.z, bottom.w};
  float otop[4], obot[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    /* pixel 4t + i lies in block 2t + i / 2 at dx = i % 2: windows at columns c0 .. c1 */
    const int c1 = 1 + i / 2;
    const int c0 = (i % 2 == 0) ? c1 - 1 : c1;
    float vt = 0.0f, vb = 0.0f;
#pragma unroll
    for (int jy = 1; jy >= 0; --jy) {  // py ascending; the row below (dy = 1) is covered by py = a only
#pragma unroll
      for (int c = c0; c <= c1; ++c) {  // px ascending
        const float tt = vt + Op::Grad(vtop[i], pv[jy][c]) * gv[jy][c];
        vt = ok[jy][c] ? tt : vt;
        if (jy == 0) {
          const float tb = vb + Op::Grad(vbot[i], pv[jy][c]) * gv[jy][c];
          vb = ok[jy][c] ? tb : vb;
        }
      }
    }
    otop[i] = vt;
    obot[i] = vb;
  }
  float *out = dst + (static_cast<size_t>(plane) * g.h + 2 * a) * dstride + 4u * t;
  F4 q;
  if (!RAGGED) {
    q.x = otop[0], q.y = otop[1], q.z = otop[2], q.w = otop[3];
    StreamStoreF4(out, q);
    q.x = obot[0], q.y = obot[1], q.z = obot[2], q.w = obot[3];
    StreamStoreF4(out + dstride, q);
  } else if (live_px == 4) {
    q.x = otop[0], q.y = otop[1], q.z = otop[2], q.w = otop[3];
    StreamStoreF4Anywhere(out, q);
    q.x = obot[0], q.y = obot[1], q.z = obot[2], q.w = obot[3];
    if (has_bottom) StreamStoreF4Anywhere(out + dstride, q);
  } else {
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      if (i < live_px) {
        StreamStore(out + i, otop[i]);
        if (has_bottom) StreamStore(out + dstride + i, obot[i]);
      }
    }
  }
}

/*! \brief geometry of the stride-1 kernels below: a plane is cut into strips of `strip_rows`
 *  rows; a strip is `groups` = ceil(w / 4) lanes wide and a wave takes `strips_per_wave`
 *  consecutive strips (plane after plane), whole rows each */
struct SlideGeom {
  uint32_t groups, strips_per_wave, strip_rows, strips_per_plane, total_strips;
  mshadow::FastDivU32 div_groups, div_spp;
  size_t src_floats, pooled_floats, grad_floats;  //!< extent of each input, last row unpadded (4 or more)
};

/*! \brief the four floats at `p` as one 16-byte access at any alignment, with no branch around
 *  the load (a loop that keeps several rows on their way needs every path to issue the same
 *  loads, or the compiler waits for all of them at every use). Where `ok` is false the pack is
 *  fetched from `base` instead and means nothing. Only the last pack of a tensor's last row can
 *  reach past the tensor's end (`end`: one past its last float): it is fetched from end - 4 and
 *  its elements are moved into place, zeros behind them. Floats past the end of a ROW are the
 *  next row's and are the caller's to ignore or mask. */
__device__ __forceinline__ F4 LoadPackFree(const float *base, const float *p, const float *end, bool ok) {
  const float *last = end - 4;
  const bool moved = ok && p > last;
  const float *at = ok ? (moved ? last : p) : base;
  F4 q = StreamLoadF4Anywhere(at);
  if (__any(moved)) {  // one wave of the grid at most
    const int sh = moved ? static_cast<int>(p - last) : 0;
    F4 b, c;
    b[0] = (sh & 1) ? q[1] : q[0];
    b[1] = (sh & 1) ? q[2] : q[1];
    b[2] = (sh & 1) ? q[3] : q[2];
    b[3] = (sh & 1) ? 0.0f : q[3];
    c[0] = (sh & 2) ? b[2] : b[0];
    c[1] = (sh & 2) ? b[3] : b[1];
    c[2] = (sh & 2) ? 0.0f : b[2];
    c[3] = (sh & 2) ? 0.0f : b[3];
#pragma unroll
    for (int e = 0; e < 4; ++e) q[e] = sh >= 4 ? 0.0f : c[e];
  }
  return q;
}
/*! \brief q with zeros in the columns from n on (and everywhere unless ok) */
__device__ __forceinline__ F4 KeepColumns(F4 q, int x0, int n, bool ok) {
#pragma unroll
  for (int e = 0; e < 4; ++e) q[e] = (ok && x0 + e < n) ? q[e] : 0.0f;
  return q;
}

/*! \brief value of v in the lane below; lane 0 receives 0 */
__device__ __forceinline__ float FromLaneBelow(float v) {
  return __uint_as_float(static_cast<uint32_t>(
      __builtin_amdgcn_update_dpp(0, static_cast<int>(__float_as_uint(v)), 0x138, 0xf, 0xf, false)));
}

/*! \brief unpool for K x K windows with stride 1 (K = 2, 3) on rows of up to 256 pixels, with no
 *  staging. A pixel lies under up to K * K windows, so a thread that took its pooled values from
 *  memory pixel by pixel would fetch every one of them K * K times. Here a thread owns four
 *  adjacent pixels and walks down a strip of rows with the K pooled rows that cover the current
 *  source row in registers: per source row it fetches one pack of the source, one of the pooled
 *  values and one of the gradients (the new pooled row; the K - 1 columns to the left of its own
 *  four come from the neighbouring lane, which holds them as its own), computes its four pixels
 *  from the K x (K + 3) windows it holds, and stores one pack. Every byte is fetched once apart
 *  from the K - 1 pooled rows on top of a strip; DEPTH rows are on their way while one is
 *  computed. The loop is unrolled DEPTH times (a multiple of K), so the K window rows are a ring
 *  of registers with fixed places: pooled row py sits in ring row (py - y0) mod K.
 *
 *  The kernel is bound by its arithmetic (K * K terms per pixel), so a term is three
 *  instructions: the reference adds PartialGrad(src, pooled) * grad, a product that is grad
 *  where the two are equal and 0 * grad where not (a zero with grad's sign, NaN for an infinite
 *  grad); Z = 0 * grad is made once per gradient fetched and the term is picked from (grad, Z)
 *  (for K = 5 the product is made per term instead: a third array of 40 registers would leave
 *  one wave per SIMD).
 *  Windows that do not exist (outside the pooled grid) are held as gradient 0: their term is
 *  +0, and adding a zero never changes the sum, which starts at +0 and so is never -0. The terms
 *  are added in the reference's order (py, then px ascending; mshadow/extension/
 *  spatial_unpool.h:102-125). */
template <int REDUCER, int K, int DEPTH>
__global__ void __launch_bounds__(kPoolBlock)
    UnpoolSlideS1Kernel(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                        int pstride, const float *grad, int gstride, PoolGeom g, SlideGeom sg) {
  static_assert(DEPTH % K == 0, "the ring of window rows must close within one unrolled turn");
  const int WIN = K + 3;  // window columns x0 - (K - 1) .. x0 + 3
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = blockIdx.x * (kPoolBlock / 64) + (threadIdx.x >> 6);
  const uint32_t sub = sg.div_groups.Div(lane);
  const uint32_t t = lane - sub * sg.groups;
  const uint32_t strip = wave * sg.strips_per_wave + sub;
  const bool live = sub < sg.strips_per_wave && strip < sg.total_strips;
  const uint32_t stripc = live ? strip : sg.total_strips - 1u;
  const uint32_t plane = sg.div_spp.Div(stripc);
  const int y0 = static_cast<int>((stripc - plane * sg.strips_per_plane) * sg.strip_rows);
  const int x0 = static_cast<int>(4u * t);
  const float *pbase = pooled + static_cast<size_t>(plane) * g.ph * pstride;
  const float *gbase = grad + static_cast<size_t>(plane) * g.ph * gstride;
  const float *sbase = src + static_cast<size_t>(plane) * g.h * sstride;
  float *dbase = dst + static_cast<size_t>(plane) * g.h * dstride;
  const float *send = src + sg.src_floats, *pend = pooled + sg.pooled_floats, *gend = grad + sg.grad_floats;
  float P[K][WIN], G[K][WIN], Z[K][WIN];
  /* a pooled row takes its place in the ring (every lane of the wave takes part) */
#define MSHADOW_SLIDE_PUT(SLOT, pq, gq)                                     \
  {                                                                         \
    _Pragma("unroll") for (int e = 0; e < 4; ++e) {                         \
      P[SLOT][K - 1 + e] = (pq)[e];                                         \
      G[SLOT][K - 1 + e] = (gq)[e];                                         \
    }                                                                       \
    _Pragma("unroll") for (int i = 0; i + 1 < K; ++i) {                     \
      const float pl = FromLaneBelow(P[SLOT][4 + i]);                       \
      const float gl = FromLaneBelow(G[SLOT][4 + i]);                       \
      P[SLOT][i] = pl;                                                      \
      G[SLOT][i] = t == 0u ? 0.0f : gl;                                     \
    }                                                                       \
    if (K <= 3) {                                                           \
      _Pragma("unroll") for (int i = 0; i < WIN; ++i) Z[SLOT][i] = 0.0f * G[SLOT][i]; \
    }                                                                       \
  }
  /* the K - 1 pooled rows above the strip's first source row: row y0 - k in ring row K - k */
#pragma unroll
  for (int k = K - 1; k >= 1; --k) {
    const int py = y0 - k;
    const bool ok = live && py >= 0 && py < g.ph;
    const F4 pq = LoadPackFree(pbase, pbase + static_cast<ptrdiff_t>(py) * pstride + x0, pend, ok);
    const F4 gq = KeepColumns(LoadPackFree(gbase, gbase + static_cast<ptrdiff_t>(py) * gstride + x0, gend, ok),
                              x0, g.pw, ok);
    MSHADOW_SLIDE_PUT(K - k, pq, gq)
  }
  const int rows = static_cast<int>(sg.strip_rows);  // the same for every lane of the wave
  F4 sq[DEPTH], pq[DEPTH], gq[DEPTH];
  bool okq[DEPTH];
#pragma unroll
  for (int u = 0; u < DEPTH; ++u) {
    const int y = y0 + u;
    okq[u] = live && u < rows && y < g.h;
    const bool pok = okq[u] && y < g.ph;
    sq[u] = LoadPackFree(sbase, sbase + static_cast<size_t>(y) * sstride + x0, send, okq[u]);
    pq[u] = LoadPackFree(pbase, pbase + static_cast<size_t>(y) * pstride + x0, pend, pok);
    gq[u] = KeepColumns(LoadPackFree(gbase, gbase + static_cast<size_t>(y) * gstride + x0, gend, pok), x0, g.pw, pok);
  }
  for (int r0 = 0; r0 < rows; r0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const int r = r0 + u;
      if (r >= rows) break;  // the same for every lane
      const int y = y0 + r;
      const F4 cur = sq[u];
      const bool cur_ok = okq[u];
      MSHADOW_SLIDE_PUT(u % K, pq[u], gq[u])
      const int yn = y + DEPTH;
      okq[u] = live && r + DEPTH < rows && yn < g.h;
      const bool pok = okq[u] && yn < g.ph;
      sq[u] = LoadPackFree(sbase, sbase + static_cast<size_t>(yn) * sstride + x0, send, okq[u]);
      pq[u] = LoadPackFree(pbase, pbase + static_cast<size_t>(yn) * pstride + x0, pend, pok);
      gq[u] = KeepColumns(LoadPackFree(gbase, gbase + static_cast<size_t>(yn) * gstride + x0, gend, pok), x0, g.pw, pok);
      F4 out;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float val = 0.0f;
#pragma unroll
        for (int k = 0; k < K; ++k) {      // py = y - (K - 1) + k, in ring row (u + 1 + k) % K
          const int slot = (u + 1 + k) % K;
#pragma unroll
          for (int j = 0; j < K; ++j) {    // px = x - (K - 1) + j
            const bool hit = REDUCER == MSHADOW_HIP_SUM || cur[e] == P[slot][e + j];
            val = val + (hit ? G[slot][e + j] : (K <= 3 ? Z[slot][e + j] : 0.0f * G[slot][e + j]));
          }
        }
        out[e] = val;
      }
      if (cur_ok) {
        float *orow = dbase + static_cast<size_t>(y) * dstride + x0;
        if (x0 + 4 <= g.w) {
          StreamStoreF4Anywhere(orow, out);
        } else {
#pragma unroll
          for (int e = 0; e < 3; ++e) {
            if (x0 + e < g.w) StreamStore(orow + e, out[e]);
          }
        }
      }
    }
  }
#undef MSHADOW_SLIDE_PUT
}

/*! \brief unpool without staging */
template <int REDUCER>
__global__ void __launch_bounds__(kPoolBlock)
    UnpoolDirectKernel(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                       int pstride, const float *grad, int gstride, PoolGeom g, unsigned total) {
  typedef PoolOp<REDUCER> Op;
  for (unsigned o = blockIdx.x * kPoolBlock + threadIdx.x; o < total; o += gridDim.x * kPoolBlock) {
    const unsigned i = o / g.w;
    const int x = o - i * g.w;
    const int y = i % g.h;
    const int plane = i / g.h;
    const float vsrc = src[static_cast<size_t>(i) * sstride + x];
    const int py_min = y < g.ky ? 0 : (y - g.ky + g.sy) / g.sy;
    const int px_min = x < g.kx ? 0 : (x - g.kx + g.sx) / g.sx;
    const int py_max = min((y + g.sy) / g.sy, g.ph);
    const int px_max = min((x + g.sx) / g.sx, g.pw);
    float val = 0.0f;
    for (int py = py_min; py < py_max; ++py) {
      const size_t prow = static_cast<size_t>(plane) * g.ph + py;
      for (int px = px_min; px < px_max; ++px) {
        val = val + Op::Grad(vsrc, pooled[prow * pstride + px]) * grad[prow * gstride + px];
      }
    }
    dst[static_cast<size_t>(i) * dstride + x] = val;
  }
}

}  // namespace mshadow_hipk
#endif  // MSHADOW_AMD_CSRC_POOL_KERNELS_H_
