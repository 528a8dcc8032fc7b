/*
 * Pooling forward / backward over the last two dimensions, LDS-tiled.
 *
 * The reference evaluates pool / unpool through its generic map kernel with
 * Plan<PoolingExp>::Eval / Plan<UnPoolingExp>::Eval as the body
 * (mshadow/extension/spatial_pool.h:125-142, spatial_unpool.h:102-125), i.e. ky*kx
 * scattered global loads per output. Here a workgroup stages a band of input rows of
 * one (n, c) plane in LDS with coalesced loads and every window is then read from LDS,
 * so HBM sees each input element once:
 *   pool    reads  planes*h*w*4 B, writes planes*ph*pw*4 B
 *   unpool  reads  planes*(h*w + 2*ph*pw)*4 B, writes planes*h*w*4 B
 * Results are bit-identical to the reference: same window clipping, same (y, x)
 * reduction order from the reducer's initial value, `max` / `min` by operator<, and the
 * gradient routed by equality with a separate multiply and add (no fused multiply-add).
 */
#ifndef MSHADOW_AMD_CSRC_POOL_KERNELS_H_
#define MSHADOW_AMD_CSRC_POOL_KERNELS_H_

#include <hip/hip_runtime.h>
#include <mshadow_hip.h>

#include <cfloat>

namespace mshadow_hipk {

const int kPoolBlock = 256;

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

/*! \brief grid.x = planes * bands. Dynamic LDS: in_rows * lds_pitch floats, where
 *  in_rows = (band - 1) * sy + ky. */
template <int REDUCER>
__global__ void __launch_bounds__(kPoolBlock)
    PoolKernel(float *dst, int dstride, const float *src, int sstride, PoolGeom g) {
  extern __shared__ float smem[];
  typedef PoolOp<REDUCER> Op;
  const int plane = blockIdx.x / g.bands;
  const int band = blockIdx.x - plane * g.bands;
  const int py0 = band * g.band;
  const int npy = min(g.band, g.ph - py0);
  const int y0 = py0 * g.sy;
  const int y1 = min(y0 + (npy - 1) * g.sy + g.ky, g.h);  // one past the last row needed
  const int nrows = max(y1 - y0, 0);
  const float *in = src + (static_cast<size_t>(plane) * g.h + y0) * sstride;
  /* stage rows y0..y1 (whole width) */
  const int total = nrows * g.w;
  for (int i = threadIdx.x; i < total; i += kPoolBlock) {
    const int r = i / g.w;
    const int c = i - r * g.w;
    smem[r * g.lds_pitch + c] = in[static_cast<size_t>(r) * sstride + c];
  }
  __syncthreads();
  float *out = dst + (static_cast<size_t>(plane) * g.ph + py0) * dstride;
  const int nout = npy * g.pw;
  for (int o = threadIdx.x; o < nout; o += kPoolBlock) {
    const int py = o / g.pw;
    const int px = o - py * g.pw;
    const int ys = py * g.sy;                      // relative to y0
    const int ye = min(ys + g.ky, g.h - y0);
    const int xs = px * g.sx;
    const int xe = min(xs + g.kx, g.w);
    float res = Op::Init();
    for (int y = ys; y < ye; ++y) {
      for (int x = xs; x < xe; ++x) res = Op::Reduce(res, smem[y * g.lds_pitch + x]);
    }
    out[static_cast<size_t>(py) * dstride + px] = res;
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
 *  grad) of prow_max * lds_pitch floats, prow_max = (band + ky - 2) / sy + 2. */
template <int REDUCER>
__global__ void __launch_bounds__(kPoolBlock)
    UnpoolKernel(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                 int pstride, const float *grad, int gstride, PoolGeom g, int prow_max) {
  extern __shared__ float smem[];
  typedef PoolOp<REDUCER> Op;
  float *sp = smem;
  float *sg = smem + prow_max * g.lds_pitch;
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
  const int total = np * g.pw;
  for (int i = threadIdx.x; i < total; i += kPoolBlock) {
    const int r = i / g.pw;
    const int c = i - r * g.pw;
    sp[r * g.lds_pitch + c] = pin[static_cast<size_t>(r) * pstride + c];
    sg[r * g.lds_pitch + c] = gin[static_cast<size_t>(r) * gstride + c];
  }
  __syncthreads();
  const float *in = src + (static_cast<size_t>(plane) * g.h + y0) * sstride;
  float *out = dst + (static_cast<size_t>(plane) * g.h + y0) * dstride;
  const int nout = ny * g.w;
  for (int o = threadIdx.x; o < nout; o += kPoolBlock) {
    const int yr = o / g.w;
    const int x = o - yr * g.w;
    const int y = y0 + yr;
    const float vsrc = in[static_cast<size_t>(yr) * sstride + x];
    const int py_min = y < g.ky ? 0 : (y - g.ky + g.sy) / g.sy;
    const int px_min = x < g.kx ? 0 : (x - g.kx + g.sx) / g.sx;
    const int py_max = min((y + g.sy) / g.sy, g.ph);
    const int px_max = min((x + g.sx) / g.sx, g.pw);
    float val = 0.0f;
    for (int py = py_min; py < py_max; ++py) {
      for (int px = px_min; px < px_max; ++px) {
        const int li = (py - p0) * g.lds_pitch + px;
        val = val + Op::Grad(vsrc, sp[li]) * sg[li];
      }
    }
    out[static_cast<size_t>(yr) * dstride + x] = val;
  }
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
