/*
 * im2col / col2im (unpack_patch2col over pad, crop over pack_col2patch) for gfx950.
 *
 * Index conventions are the reference's (mshadow/extension/unpack_patch2col.h:126-141,
 * pad.h:87-99, pack_col2patch.h:118-144, crop.h:103-110):
 *   col[(c*ky + a)*kx + b][(n*OH + oy)*OW + ox] = padded_img[n][c][oy*sy + a*dy][ox*sx + b*dx]
 * and col2im adds, for an image pixel, the covering patches in (py, px) ascending order
 * in the element type (binary16 rounds after every add), then crops the padding away.
 * Both are pure data movement, HBM-bound: the column matrix (ky*kx times the image) is
 * written (im2col) or read (col2im) exactly once with contiguous accesses along the
 * column index; the image side is small and is served from cache.
 *
 * T is the storage type (uint16_t for binary16 bits, float); col2im accumulates through
 * Acc<T>, which rounds to T after each addition.
 */
#ifndef MSHADOW_AMD_CSRC_PATCH_KERNELS_H_
#define MSHADOW_AMD_CSRC_PATCH_KERNELS_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mshadow_hipk {

const int kPatchBlock = 256;

struct PatchGeom {
  int n, c, h, w;          // unpadded image
  int ky, kx, sy, sx, dy, dx;
  int pad_y, pad_x;
  int hp, wp;              // padded height / width
  int oh, ow;              // patch grid
};

template <typename T>
struct Acc;
template <>
struct Acc<float> {
  __device__ static float Zero() { return 0.0f; }
  __device__ static float Add(float a, float b) { return a + b; }
};
template <>
struct Acc<uint16_t> {
  __device__ static uint16_t Zero() { return 0; }
  __device__ static uint16_t Add(uint16_t a, uint16_t b) {
    _Float16 x, y;
    __builtin_memcpy(&x, &a, 2);
    __builtin_memcpy(&y, &b, 2);
    /* widen, add in float, round to nearest even back to binary16 */
    const _Float16 r = static_cast<_Float16>(static_cast<float>(x) + static_cast<float>(y));
    uint16_t o;
    __builtin_memcpy(&o, &r, 2);
    return o;
  }
};

/*! \brief EPT consecutive column-matrix elements per thread; grid.x = rows of the column
 *  matrix (c, a, b) times `chunks` pieces of kPatchBlock * EPT columns each. */
template <typename T, int EPT>
__global__ void __launch_bounds__(kPatchBlock)
    Im2ColKernel(T *col, int cstride, const T *img, int istride, PatchGeom g, unsigned chunks) {
  const int i = blockIdx.x / chunks;
  const int piece = blockIdx.x - i * chunks;
  const int b = (i % g.kx) * g.dx;
  const int irest = i / g.kx;
  const int a = (irest % g.ky) * g.dy;
  const int ch = irest / g.ky;
  const int ncols = g.n * g.oh * g.ow;
  const int j0 = (piece * kPatchBlock + threadIdx.x) * EPT;
  if (j0 >= ncols) return;
  int ox = j0 % g.ow;
  int jrest = j0 / g.ow;
  int oy = jrest % g.oh;
  int n = jrest / g.oh;
  T vals[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    T v = 0;
    if (j0 + e < ncols) {
      /* coordinates in the padded image; outside the stored image reads as zero */
      const int y = oy * g.sy + a - g.pad_y;
      const int x = ox * g.sx + b - g.pad_x;
      if (y >= 0 && y < g.h && x >= 0 && x < g.w) {
        v = img[(static_cast<size_t>(n * g.c + ch) * g.h + y) * istride + x];
      }
    }
    vals[e] = v;
    if (++ox == g.ow) {
      ox = 0;
      if (++oy == g.oh) {
        oy = 0;
        ++n;
      }
    }
  }
  T *out = col + static_cast<size_t>(i) * cstride + j0;
  const bool vec_ok = (j0 + EPT <= ncols) &&
                      (reinterpret_cast<uintptr_t>(out) % (sizeof(T) * EPT) == 0);
  if (vec_ok) {
    typedef T Vec __attribute__((ext_vector_type(EPT)));
    Vec pack;
#pragma unroll
    for (int e = 0; e < EPT; ++e) pack[e] = vals[e];
    *reinterpret_cast<Vec *>(out) = pack;
  } else {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      if (j0 + e < ncols) out[e] = vals[e];
    }
  }
}

/*! \brief one image pixel per thread; consecutive threads take consecutive x so that,
 *  for a fixed patch offset, their column-matrix reads are consecutive too */
template <typename T>
__global__ void __launch_bounds__(kPatchBlock)
    Col2ImKernel(T *img, int istride, const T *col, int cstride, PatchGeom g, unsigned total) {
  const int span_y = g.dy * (g.ky - 1) + 1;
  const int span_x = g.dx * (g.kx - 1) + 1;
  for (unsigned o = blockIdx.x * kPatchBlock + threadIdx.x; o < total;
       o += gridDim.x * kPatchBlock) {
    const unsigned row = o / g.w;      // (n*c + ch)*h + cy
    const int cx = o - row * g.w;
    const int cy = row % g.h;
    const unsigned plane = row / g.h;
    const int ch = plane % g.c;
    const int n = plane / g.c;
    const int y = cy + g.pad_y;        // position in the padded image
    const int x = cx + g.pad_x;
    const int py_min = y < span_y ? y % g.dy : (y - span_y + g.sy) / g.sy;
    const int px_min = x < span_x ? x % g.dx : (x - span_x + g.sx) / g.sx;
    const int py_max = min((y + g.sy) / g.sy, g.oh);
    const int px_max = min((x + g.sx) / g.sx, g.ow);
    T res = Acc<T>::Zero();
    for (int py = py_min; py < py_max; py += g.dy) {
      for (int px = px_min; px < px_max; px += g.dx) {
        const int r = (ch * g.ky + (y - py * g.sy) / g.dy) * g.kx + (x - px * g.sx) / g.dx;
        const int q = (n * g.oh + py) * g.ow + px;
        res = Acc<T>::Add(res, col[static_cast<size_t>(r) * cstride + q]);
      }
    }
    img[static_cast<size_t>(row) * istride + cx] = res;
  }
}

}  // namespace mshadow_hipk
#endif  // MSHADOW_AMD_CSRC_PATCH_KERNELS_H_
