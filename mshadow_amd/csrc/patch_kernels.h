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

#include <mshadow/core/fastdiv.h>

#include "stream_access.h"

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

/* ---------------------------------------------------------------- LDS-tiled versions
 * One workgroup per (image, channel) plane, or per band of rows of it:
 *   im2col  stages the zero-padded input band once, then writes the ky*kx shifted copies
 *           (each a contiguous run of the column matrix) with 128-bit stores;
 *   col2im  stages, per kernel tap, the contiguous run of the column matrix that the band
 *           needs (128-bit loads), then sums each pixel's covering patches from LDS in
 *           the reference's (py, px) order.
 * So the large side (the column matrix) moves through HBM exactly once in long
 * contiguous pieces and the small side once per band. */
struct PatchTile {
  int band;       // im2col: patch rows (oy) per workgroup; col2im: image rows per workgroup
  int bands;      // bands per plane
  int rows_max;   // im2col: padded input rows staged; col2im: patch rows (py) staged per tap
  int pitch;      // im2col: LDS elements per staged input row; col2im: per staged tap
};

/*! \brief which (image, channel, band) a workgroup works on: bands fastest, then images, then
 *  channels. A row of the column matrix holds one tap of one channel for all images one after
 *  the other, so workgroups that run at the same time write (or read) neighbouring stretches
 *  of the same few rows instead of one stretch in each of thousands of rows; measured on the
 *  (32,256,56,56) binary16 case, channels fastest against images fastest: im2col 99 -> 91 us. */
__device__ __forceinline__ void PlaneOfBlock(const PatchGeom &g, const PatchTile &t, int *n, int *ch,
                                             int *band) {
  const int seq = blockIdx.x / t.bands;
  *band = blockIdx.x - seq * t.bands;
  *ch = seq / g.n;
  *n = seq - *ch * g.n;
}

template <typename T, int EPT>
__global__ void __launch_bounds__(kPatchBlock)
    Im2ColTiledKernel(T *col, int cstride, const T *img, int istride, PatchGeom g, PatchTile t) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T *lds = reinterpret_cast<T *>(smem_raw);
  int n, ch, band;
  PlaneOfBlock(g, t, &n, &ch, &band);
  const int plane = n * g.c + ch;
  const int oy0 = band * t.band;
  const int noy = min(t.band, g.oh - oy0);
  const int iy0 = oy0 * g.sy;                  // first padded input row of the band
  const int in_rows = (noy - 1) * g.sy + (g.ky - 1) * g.dy + 1;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T *src = img + static_cast<size_t>(plane) * g.h * istride;
  for (int r = wave; r < in_rows; r += kPatchBlock / 64) {
    const int y = iy0 + r - g.pad_y;
    const bool row_ok = y >= 0 && y < g.h;
    for (int xx = lane; xx < g.wp; xx += 64) {
      const int x = xx - g.pad_x;
      T v = 0;
      if (row_ok && x >= 0 && x < g.w) v = src[static_cast<size_t>(y) * istride + x];
      lds[r * t.pitch + xx] = v;
    }
  }
  __syncthreads();
  /* each tap (a, b) owns one row of the column matrix and, inside it, the band is one
     contiguous run of `count` elements. A thread walks that run in packs of EPT; its
     (oy, ox) position advances by a fixed step, so the only division is the one below. */
  const int count = noy * g.ow;
  const int step = kPatchBlock * EPT;
  const int step_oy = step / g.ow;
  const int step_ox = step - step_oy * g.ow;
  const int first = threadIdx.x * EPT;
  const int first_oy = first / g.ow;
  const int first_ox = first - first_oy * g.ow;
  const size_t j0 = (static_cast<size_t>(n) * g.oh + oy0) * g.ow;
  for (int a = 0; a < g.ky; ++a) {
    for (int b = 0; b < g.kx; ++b) {
      T *row = col + static_cast<size_t>((ch * g.ky + a) * g.kx + b) * cstride + j0;
      const T *tap = lds + a * g.dy * t.pitch + b * g.dx;
      int oy = first_oy, ox = first_ox;
      for (int e0 = first; e0 < count; e0 += step) {
        T vals[EPT];
        if (ox + EPT <= g.ow) {  // the pack stays inside one patch row
          const T *p = tap + oy * g.sy * t.pitch + ox * g.sx;
#pragma unroll
          for (int e = 0; e < EPT; ++e) vals[e] = p[e * g.sx];
        } else {
          int yy = oy, xx = ox;
#pragma unroll
          for (int e = 0; e < EPT; ++e) {
            vals[e] = (e0 + e < count) ? tap[yy * g.sy * t.pitch + xx * g.sx] : static_cast<T>(0);
            if (++xx == g.ow) {
              xx = 0;
              ++yy;
            }
          }
        }
        T *out = row + e0;
        if (e0 + EPT <= count && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
          U4 pack;  // EPT elements are exactly 16 bytes
          __builtin_memcpy(&pack, vals, 16);
          StreamStore16(out, pack);
        } else {
#pragma unroll
          for (int e = 0; e < EPT; ++e) {
            if (e0 + e < count) out[e] = vals[e];
          }
        }
        ox += step_ox;
        oy += step_oy;
        if (ox >= g.ow) {
          ox -= g.ow;
          ++oy;
        }
      }
    }
  }
}

/*! \brief im2col with no staging at all, for three taps per row, stride 1, dilation 1 and dense
 *  images (binary16 or float) padded by one column on each side (ow == w): a thread makes the three packs (b = 0, 1, 2) of one place
 *  (a, oy, a pack of columns) of one channel from the aligned pack of image row oy + a - pad_y
 *  and the element on either side of it, and stores them. A workgroup is 256 consecutive places of one (channel,
 *  a) pair - the three rows of the column matrix are contiguous over images and patch rows -
 *  and ends after its three stores per thread, so the machine sees many small independent
 *  pieces, the form in which plain copies and fills run fastest here. The image is read
 *  ky times, the repeats from L2. MI355X, (32,256,56,56), pad 1: 92-94 us with the image
 *  coming from HBM and 78 us with the image in the memory-side cache, against 100-103 us
 *  and 86 us for a kernel that staged a plane's rows in LDS; two or four places per thread (PER) are slower
 *  (111 / 115 us), as is one thread storing all nine packs that one image pack feeds (125 us). */
const int kIm2ColDirectPer = 1;
template <typename T, int PER>
__global__ void __launch_bounds__(kPatchBlock)
    Im2ColRow3DirectKernel(T *col, int cstride, const T *img, PatchGeom g,
                           mshadow::FastDivU32 div_ppr, mshadow::FastDivU32 div_oh,
                           uint32_t chunks, mshadow::FastDivU32 div_chunks) {
  const int EPT = 16 / sizeof(T);
  /* Workgroups are dealt to the XCDs in turn, eight at a time. The ky workgroups that read
     the same piece of the image (one per tap row a) get numbers 8 apart: they run on one XCD
     at about the same time, and its L2 fetches that piece once.
     blockIdx = ((piece / 8) * ky + a) * 8 + piece % 8, piece = ch * chunks + chunk */
  const uint32_t lane8 = blockIdx.x & 7u;
  const uint32_t turn = blockIdx.x >> 3;
  const uint32_t group = turn / static_cast<uint32_t>(g.ky);
  const int a = static_cast<int>(turn - group * g.ky);
  const uint32_t piece = group * 8 + lane8;
  const uint32_t ch = div_chunks.Div(piece);
  if (ch >= static_cast<uint32_t>(g.c)) return;
  const uint32_t chunk = piece - ch * chunks;
  const uint32_t row3 = ch * g.ky + a;
  const uint32_t ppr = static_cast<uint32_t>(g.ow) / EPT;
  const uint32_t places = static_cast<uint32_t>(g.n) * g.oh * ppr;
  U4 w03[PER], mid[PER], hi[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const uint32_t pk = (chunk * PER + u) * kPatchBlock + threadIdx.x;
    w03[u] = mid[u] = hi[u] = U4{0u, 0u, 0u, 0u};
    if (pk >= places) continue;
    const uint32_t line = div_ppr.Div(pk);             // n * oh + oy
    const int ox = static_cast<int>(pk - line * ppr) * EPT;
    const uint32_t n = div_oh.Div(line);
    const int oy = static_cast<int>(line - n * g.oh);
    const int y = oy + a - g.pad_y;
    if (y >= 0 && y < g.h) {
      const T *in = img + (static_cast<size_t>(n * g.c + ch) * g.h + y) * g.w + ox;
      const U4 m = *reinterpret_cast<const U4 *>(in);
      uint32_t before = 0u, after = 0u;                // the element on either side, zero-extended
      if (ox > 0) __builtin_memcpy(&before, in - 1, sizeof(T));
      if (ox + EPT < g.w) __builtin_memcpy(&after, in + EPT, sizeof(T));
      mid[u] = m;
      if (sizeof(T) == 2) {
        w03[u].x = (m.x << 16) | before;
        w03[u].y = __builtin_amdgcn_alignbit(m.y, m.x, 16);
        w03[u].z = __builtin_amdgcn_alignbit(m.z, m.y, 16);
        w03[u].w = __builtin_amdgcn_alignbit(m.w, m.z, 16);
        hi[u].x = w03[u].y;
        hi[u].y = w03[u].z;
        hi[u].z = w03[u].w;
        hi[u].w = (after << 16) | (m.w >> 16);
      } else {
        w03[u] = U4{before, m.x, m.y, m.z};
        hi[u] = U4{m.y, m.z, m.w, after};
      }
    }
  }
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const uint32_t pk = (chunk * PER + u) * kPatchBlock + threadIdx.x;
    if (pk >= places) continue;
    T *out = col + static_cast<size_t>(row3 * 3) * cstride + static_cast<size_t>(pk) * EPT;
    StreamStore16(out, w03[u]);
    StreamStore16(out + cstride, mid[u]);
    StreamStore16(out + 2 * static_cast<size_t>(cstride), hi[u]);
  }
}

/* ------------------------------------------------------- stride 1, dilation 1, any window
 * With stride and dilation 1 the row (channel, a, b) of the column matrix is, image by image,
 * the image itself shifted by (a - pad_y, b - pad_x) and cut to the patch grid: a run of a
 * patch row is a run of an image row. So both directions can work pack by pack with no
 * staging: one side of a pack is aligned (the side that is stored), the other is fetched
 * wherever it lies - 16-byte global loads need no alignment on this machine. Very many small
 * workgroups that end after a handful of accesses each. */

/*! \brief 16 bytes from an address aligned only to the element */
template <typename T>
__device__ __forceinline__ U4 LoadPackAnywhere(const T *p) {
  typedef U4 Loose __attribute__((aligned(2)));   // the narrowest element type here
  return *reinterpret_cast<const Loose *>(p);
}

/*! \brief element e of a pack of EPT elements of type T, and its replacement */
template <typename T>
__device__ __forceinline__ T PackElement(const U4 &q, int e) {
  const int per = 4 / sizeof(T);   // elements per dword
  const uint32_t w = q[e / per];
  T v;
  if (sizeof(T) == 4) {
    __builtin_memcpy(&v, &w, sizeof(T));
  } else {
    const uint16_t h = static_cast<uint16_t>(w >> (16 * (e % per)));
    __builtin_memcpy(&v, &h, sizeof(T));
  }
  return v;
}
template <typename T>
__device__ __forceinline__ void SetPackElement(U4 *q, int e, T v) {
  const int per = 4 / sizeof(T);
  if (sizeof(T) == 4) {
    uint32_t w;
    __builtin_memcpy(&w, &v, 4);
    (*q)[e / per] = w;
  } else {
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    const int sh = 16 * (e % per);
    (*q)[e / per] = ((*q)[e / per] & ~(0xffffu << sh)) | (static_cast<uint32_t>(h) << sh);
  }
}

template <typename T>
__device__ __forceinline__ void StorePackAnywhere(T *p, const U4 &q) {
  typedef U4 Loose __attribute__((aligned(2)));
  __builtin_nontemporal_store(q, reinterpret_cast<Loose *>(p));
}

/*! \brief the pack with every element outside [lo, hi) cleared */
template <typename T>
__device__ __forceinline__ U4 KeepElements(U4 q, int lo, int hi) {
  const int per = 4 / sizeof(T);
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    uint32_t m = 0u;
#pragma unroll
    for (int k = 0; k < per; ++k) {
      const int e = d * per + k;
      if (e >= lo && e < hi) m |= (sizeof(T) == 4 ? 0xffffffffu : 0xffffu << (16 * k));
    }
    q[d] &= m;
  }
  return q;
}

/*! \brief EPT consecutive elements from p, of which only [lo, hi) are wanted (the others come
 *  back as zero): one 16-byte load where all 16 bytes lie inside [first, last), else element
 *  by element */
template <typename T>
__device__ __forceinline__ U4 LoadPackInside(const T *p, int lo, int hi, const T *first, const T *last) {
  const int EPT = 16 / sizeof(T);
  if (p >= first && p + EPT <= last) return KeepElements<T>(LoadPackAnywhere(p), lo, hi);
  U4 q = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    if (e >= lo && e < hi) SetPackElement(&q, e, p[e]);
  }
  return q;
}

/*! \brief im2col, stride 1, dilation 1, patch rows of at least one pack: a thread makes one pack
 *  of one patch row of one row of the column matrix. The last pack of a patch row that is not
 *  whole packs is moved back to end with the row (it overlaps its neighbour, both write the
 *  same values), so no pack ever straddles two rows. grid: the taps of one piece of a channel 8
 *  workgroups apart, as in Im2ColRow3DirectKernel. */
template <typename T>
__global__ void __launch_bounds__(kPatchBlock)
    Im2ColDirectS1Kernel(T *col, int cstride, const T *img, int istride, PatchGeom g,
                         mshadow::FastDivU32 div_ppr, mshadow::FastDivU32 div_oh, uint32_t chunks,
                         mshadow::FastDivU32 div_chunks, uint32_t places) {
  const int EPT = 16 / sizeof(T);
  const uint32_t taps = static_cast<uint32_t>(g.ky * g.kx);
  const uint32_t lane8 = blockIdx.x & 7u;
  const uint32_t turn = blockIdx.x >> 3;
  const uint32_t group = turn / taps;
  const uint32_t tap = turn - group * taps;
  const uint32_t piece = group * 8 + lane8;
  const uint32_t ch = div_chunks.Div(piece);
  if (ch >= static_cast<uint32_t>(g.c)) return;
  const uint32_t chunk = piece - ch * chunks;
  const int a = static_cast<int>(tap) / g.kx;
  const int b = static_cast<int>(tap) - a * g.kx;
  const uint32_t pk = chunk * kPatchBlock + threadIdx.x;   // place: (n * oh + oy) * ppr + p
  if (pk >= places) return;
  const uint32_t line = div_ppr.Div(pk);
  const int ox = min(static_cast<int>(pk - line * div_ppr.div) * EPT, g.ow - EPT);
  const uint32_t n = div_oh.Div(line);
  const int oy = static_cast<int>(line - n * g.oh);
  const int y = oy + a - g.pad_y;
  const int xs = ox + b - g.pad_x;
  U4 q = {0u, 0u, 0u, 0u};
  if (y >= 0 && y < g.h) {
    const T *row = img + (static_cast<size_t>(n * g.c + ch) * g.h + y) * istride;
    const T *last = img + (static_cast<size_t>(g.n) * g.c * g.h - 1) * istride + g.w;
    q = LoadPackInside<T>(row + xs, max(0, -xs), min(EPT, g.w - xs), img, last);
  }
  StorePackAnywhere(col + static_cast<size_t>(ch * taps + tap) * cstride +
                        static_cast<size_t>(line) * g.ow + ox, q);
}

/*! \brief im2col with a step of two pixels between patches in a row (any step between rows, any
 *  dilation), patch rows of at least one pack: as Im2ColDirectS1Kernel, but the EPT pixels of a
 *  pack lie two apart in the image: the thread fetches the two packs that hold them and keeps
 *  every second element. */
template <typename T>
__global__ void __launch_bounds__(kPatchBlock)
    Im2ColDirectS2Kernel(T *col, int cstride, const T *img, int istride, PatchGeom g,
                         mshadow::FastDivU32 div_ppr, mshadow::FastDivU32 div_oh, uint32_t chunks,
                         mshadow::FastDivU32 div_chunks, uint32_t places) {
  const int EPT = 16 / sizeof(T);
  const uint32_t taps = static_cast<uint32_t>(g.ky * g.kx);
  const uint32_t lane8 = blockIdx.x & 7u;
  const uint32_t turn = blockIdx.x >> 3;
  const uint32_t group = turn / taps;
  const uint32_t tap = turn - group * taps;
  const uint32_t piece = group * 8 + lane8;
  const uint32_t ch = div_chunks.Div(piece);
  if (ch >= static_cast<uint32_t>(g.c)) return;
  const uint32_t chunk = piece - ch * chunks;
  const int a = static_cast<int>(tap) / g.kx;
  const int b = static_cast<int>(tap) - a * g.kx;
  const uint32_t pk = chunk * kPatchBlock + threadIdx.x;   // place: (n * oh + oy) * ppr + p
  if (pk >= places) return;
  const uint32_t line = div_ppr.Div(pk);
  const int ox = min(static_cast<int>(pk - line * div_ppr.div) * EPT, g.ow - EPT);
  const uint32_t n = div_oh.Div(line);
  const int oy = static_cast<int>(line - n * g.oh);
  const int y = oy * g.sy + a * g.dy - g.pad_y;
  const int xs = ox * 2 + b * g.dx - g.pad_x;
  U4 q = {0u, 0u, 0u, 0u};
  if (y >= 0 && y < g.h) {
    const T *row = img + (static_cast<size_t>(n * g.c + ch) * g.h + y) * istride;
    const T *last = img + (static_cast<size_t>(g.n) * g.c * g.h - 1) * istride + g.w;
    const U4 lo = LoadPackInside<T>(row + xs, max(0, -xs), min(EPT, g.w - xs), img, last);
    const U4 hi = LoadPackInside<T>(row + xs + EPT, max(0, -xs - EPT), min(EPT, g.w - xs - EPT), img, last);
    if (sizeof(T) == 4) {
      q[0] = lo[0], q[1] = lo[2], q[2] = hi[0], q[3] = hi[2];
    } else {
      q[0] = __builtin_amdgcn_perm(lo[1], lo[0], 0x05040100u);
      q[1] = __builtin_amdgcn_perm(lo[3], lo[2], 0x05040100u);
      q[2] = __builtin_amdgcn_perm(hi[1], hi[0], 0x05040100u);
      q[3] = __builtin_amdgcn_perm(hi[3], hi[2], 0x05040100u);
    }
  }
  StorePackAnywhere(col + static_cast<size_t>(ch * taps + tap) * cstride +
                        static_cast<size_t>(line) * g.ow + ox, q);
}

/*! \brief LoadPackInside with the one 16-byte load outside any branch (a load inside a branch
 *  makes the compiler wait for every load under way before it): the address is moved into
 *  [first, last - EPT] for the load, and only a wave that holds a moved pack - at the first or
 *  the last row of the whole tensor - fetches that pack again element by element. `wanted` false:
 *  nothing is wanted, zeros come back. */
template <typename T>
__device__ __forceinline__ U4 LoadPackInsideFree(const T *p, int lo, int hi, const T *first, const T *last,
                                                 bool wanted) {
  const int EPT = 16 / sizeof(T);
  const bool moved = wanted && (p < first || p + EPT > last);
  const T *at = !wanted ? first : (p < first ? first : (p + EPT > last ? last - EPT : p));
  U4 q = LoadPackAnywhere(at);
  if (__any(moved)) {
    U4 r = {0u, 0u, 0u, 0u};
    if (moved) {
#pragma unroll
      for (int e = 0; e < EPT; ++e) {
        if (e >= lo && e < hi) SetPackElement(&r, e, p[e]);
      }
    }
    if (moved) q = r;
  }
  return KeepElements<T>(q, wanted ? lo : 0, wanted ? hi : 0);
}

/*! \brief im2col with a step of SX = 1 or 2 between patches in a row and dilation 1 along the
 *  row, for KX taps a row (3, 4, 5 or 7): a thread makes the packs of ALL KX taps of one tap row
 *  at one place from the SX * (EPT - 1) + KX neighbouring image elements under them, fetched
 *  once as two to four packs (Im2ColDirectS1Kernel fetches a pack per tap, Im2ColDirectS2Kernel
 *  two: the image then crosses from L2 to the CUs KX or 2 * KX times per tap row). Tap b's pack
 *  is every SX-th element from the b-th on. The tap rows of one piece of a channel are numbered
 *  8 workgroups apart, as in Im2ColRow3DirectKernel. */
template <typename T, int KX, int SX>
__global__ void __launch_bounds__(kPatchBlock)
    Im2ColRowTapsKernel(T *col, int cstride, const T *img, int istride, PatchGeom g,
                        mshadow::FastDivU32 div_ppr, mshadow::FastDivU32 div_oh, uint32_t chunks,
                        mshadow::FastDivU32 div_chunks, uint32_t places) {
  const int EPT = 16 / sizeof(T);
  const int NPACK = (SX * (EPT - 1) + KX + EPT - 1) / EPT;
  const uint32_t rows = static_cast<uint32_t>(g.ky);
  const uint32_t lane8 = blockIdx.x & 7u;
  const uint32_t turn = blockIdx.x >> 3;
  const uint32_t group = turn / rows;
  const int a = static_cast<int>(turn - group * rows);
  const uint32_t piece = group * 8 + lane8;
  const uint32_t ch = div_chunks.Div(piece);
  if (ch >= static_cast<uint32_t>(g.c)) return;
  const uint32_t chunk = piece - ch * chunks;
  const uint32_t pk = chunk * kPatchBlock + threadIdx.x;   // place: (n * oh + oy) * ppr + p
  if (pk >= places) return;
  const uint32_t line = div_ppr.Div(pk);
  const int ox = min(static_cast<int>(pk - line * div_ppr.div) * EPT, g.ow - EPT);
  const uint32_t n = div_oh.Div(line);
  const int oy = static_cast<int>(line - n * g.oh);
  const int y = oy * g.sy + a * g.dy - g.pad_y;
  const int xs = ox * SX - g.pad_x;
  const bool wanted = y >= 0 && y < g.h;
  const T *row = img + (static_cast<size_t>(n * g.c + ch) * g.h + (wanted ? y : 0)) * istride;
  const T *last = img + (static_cast<size_t>(g.n) * g.c * g.h - 1) * istride + g.w;
  uint32_t R[NPACK * 4];
#pragma unroll
  for (int k = 0; k < NPACK; ++k) {
    const int at = xs + k * EPT;
    const U4 q = LoadPackInsideFree<T>(row + at, max(0, -at), min(EPT, g.w - at), img, last, wanted);
#pragma unroll
    for (int d = 0; d < 4; ++d) R[4 * k + d] = q[d];
  }
  T *out = col + static_cast<size_t>(ch * rows * KX + a * KX) * cstride + static_cast<size_t>(line) * g.ow + ox;
#pragma unroll
  for (int b = 0; b < KX; ++b) {
    U4 q;
    if (sizeof(T) == 4) {
#pragma unroll
      for (int e = 0; e < 4; ++e) q[e] = R[SX * e + b];
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i0 = SX * 2 * r + b, i1 = i0 + SX;   // the two elements of this register
        const uint32_t lo = (i0 & 1) ? 0x0302u : 0x0100u, hi = (i1 & 1) ? 0x0706u : 0x0504u;
        q[r] = __builtin_amdgcn_perm(R[i1 >> 1], R[i0 >> 1], (hi << 16) | lo);
      }
    }
    StorePackAnywhere(out + static_cast<size_t>(b) * cstride, q);
  }
}

/*! \brief one pack plus another, element by element, rounded after every add as the element
 *  type's own += does (binary16: a packed half add is exactly that); elements whose bit in
 *  `keep` is clear stay as they are */
template <typename T>
__device__ __forceinline__ void AddPackWhere(U4 *acc, const U4 &term, uint32_t keep) {
  const int EPT = 16 / sizeof(T);
  if (sizeof(T) == 4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float x, y;
      const uint32_t xa = (*acc)[e], ya = term[e];
      __builtin_memcpy(&x, &xa, 4);
      __builtin_memcpy(&y, &ya, 4);
      const float r = x + y;
      uint32_t w;
      __builtin_memcpy(&w, &r, 4);
      if (keep & (1u << e)) (*acc)[e] = w;
    }
  } else {
    typedef _Float16 H2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      H2 x, y;
      const uint32_t xa = (*acc)[d], ya = term[d];
      __builtin_memcpy(&x, &xa, 4);
      __builtin_memcpy(&y, &ya, 4);
      const H2 r = x + y;
      uint32_t w;
      __builtin_memcpy(&w, &r, 4);
      const uint32_t m = ((keep >> (2 * d)) & 1u ? 0x0000ffffu : 0u) |
                         ((keep >> (2 * d + 1)) & 1u ? 0xffff0000u : 0u);
      (*acc)[d] = (w & m) | ((*acc)[d] & ~m);
    }
  }
  (void)EPT;
}

/*! \brief col2im, stride 1, dilation 1, image rows of at least one pack: a thread sums one pack of
 *  an image row (the last pack of a row that is not whole packs moved back to end with the
 *  row, as above) from the ky * kx rows of the column matrix that cover it, terms in the
 *  reference's order (py ascending, then px ascending:
 *  mshadow/extension/pack_col2patch.h:118-144). */
template <typename T>
__global__ void __launch_bounds__(kPatchBlock)
    Col2ImDirectS1Kernel(T *img, int istride, const T *col, int cstride, PatchGeom g,
                         mshadow::FastDivU32 div_wpk, mshadow::FastDivU32 div_h,
                         mshadow::FastDivU32 div_c, uint32_t total_packs) {
  const int EPT = 16 / sizeof(T);
  const uint32_t pk = blockIdx.x * kPatchBlock + threadIdx.x;
  if (pk >= total_packs) return;
  const uint32_t rowi = div_wpk.Div(pk);             // (n * c + ch) * h + y
  const int x0 = min(static_cast<int>(pk - rowi * div_wpk.div) * EPT, g.w - EPT);
  const uint32_t plane = div_h.Div(rowi);
  const int y = static_cast<int>(rowi - plane * g.h);
  const uint32_t n = div_c.Div(plane);
  const uint32_t ch = plane - n * g.c;
  const uint32_t taps = static_cast<uint32_t>(g.ky * g.kx);
  const size_t cols = static_cast<size_t>(g.n) * g.oh * g.ow;
  const T *last = col + (static_cast<size_t>(g.c) * taps - 1) * cstride + cols;
  const T *base = col + static_cast<size_t>(ch) * taps * cstride + static_cast<size_t>(n) * g.oh * g.ow;
  U4 acc = {0u, 0u, 0u, 0u};
  for (int a = g.ky - 1; a >= 0; --a) {
    const int py = y + g.pad_y - a;
    if (py < 0 || py >= g.oh) continue;
    for (int b = g.kx - 1; b >= 0; --b) {
      const int px0 = x0 + g.pad_x - b;              // patch column of the pack's first pixel
      const int lo = max(0, -px0), hi = min(EPT, g.ow - px0);   // elements [lo, hi) have a patch
      if (lo >= hi) continue;
      const T *at = base + static_cast<size_t>(a * g.kx + b) * cstride + static_cast<size_t>(py) * g.ow;
      const U4 term = LoadPackInside<T>(at + px0, lo, hi, col, last);
      const uint32_t keep = ((1u << hi) - 1u) & ~((1u << lo) - 1u);
      AddPackWhere<T>(&acc, term, keep);
    }
  }
  StorePackAnywhere(img + static_cast<size_t>(rowi) * istride + x0, acc);
}

/*! \brief FAST: stride 1 and dilation 1 in both directions (the common convolution case):
 *  every patch-range bound is then a subtraction instead of a division. */
template <typename T, int EPT, bool FAST>
__global__ void __launch_bounds__(kPatchBlock)
    Col2ImTiledKernel(T *img, int istride, const T *col, int cstride, PatchGeom g, PatchTile t) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T *lds = reinterpret_cast<T *>(smem_raw);
  if (FAST) {
    g.sy = g.sx = g.dy = g.dx = 1;
  }
  int n, ch, band;
  PlaneOfBlock(g, t, &n, &ch, &band);
  const int plane = n * g.c + ch;
  const int cy0 = band * t.band;
  const int ncy = min(t.band, g.h - cy0);
  const int span_y = g.dy * (g.ky - 1) + 1;
  const int span_x = g.dx * (g.kx - 1) + 1;
  /* patch rows any pixel row of the band can touch */
  const int yf = cy0 + g.pad_y, yl = cy0 + ncy - 1 + g.pad_y;
  const int p0 = yf < span_y ? 0 : (yf - span_y + g.sy) / g.sy;
  const int p1 = min((yl + g.sy) / g.sy, g.oh);
  const int npy = max(p1 - p0, 0);
  const int run = npy * g.ow;                  // contiguous column-matrix elements per tap
  const int taps = g.ky * g.kx;
  const size_t j0 = (static_cast<size_t>(n) * g.oh + p0) * g.ow;
  for (int tap = 0; tap < taps; ++tap) {
    const T *in = col + static_cast<size_t>(ch * taps + tap) * cstride + j0;
    T *out = lds + tap * t.pitch;              // t.pitch is a multiple of EPT: aligned
    const bool vec_ok = reinterpret_cast<uintptr_t>(in) % (sizeof(T) * EPT) == 0;
    for (int e0 = threadIdx.x * EPT; e0 < run; e0 += kPatchBlock * EPT) {
      if (vec_ok && e0 + EPT <= run) {
        *reinterpret_cast<U4 *>(out + e0) = StreamLoad16(in + e0);
      } else {
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
          if (e0 + e < run) out[e0 + e] = in[e0 + e];
        }
      }
    }
  }
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  T *dst = img + (static_cast<size_t>(plane) * g.h + cy0) * istride;
  for (int cyr = wave; cyr < ncy; cyr += kPatchBlock / 64) {
    const int y = cy0 + cyr + g.pad_y;
    const int py_min = y < span_y ? y % g.dy : (y - span_y + g.sy) / g.sy;
    const int py_max = min((y + g.sy) / g.sy, g.oh);
    for (int cx = lane; cx < g.w; cx += 64) {
      const int x = cx + g.pad_x;
      const int px_min = x < span_x ? x % g.dx : (x - span_x + g.sx) / g.sx;
      const int px_max = min((x + g.sx) / g.sx, g.ow);
      T res = Acc<T>::Zero();
      for (int py = py_min; py < py_max; py += g.dy) {
        const int a = (y - py * g.sy) / g.dy;
        for (int px = px_min; px < px_max; px += g.dx) {
          const int b = (x - px * g.sx) / g.dx;
          res = Acc<T>::Add(res, lds[(a * g.kx + b) * t.pitch + (py - p0) * g.ow + px]);
        }
      }
      dst[static_cast<size_t>(cyr) * istride + cx] = res;
    }
  }
}

/*! \brief geometry of Col2ImHalfRows3x3Kernel: rows of all image planes are numbered
 *  plane * h + y; a wave takes `rows_per_wave` consecutive ones, `groups` lanes per row
 *  (numbered channel by channel instead, all images of a channel together, the kernel took
 *  98 us instead of 91) */
struct RowsGeom {
  uint32_t total_rows;     //!< n * c * h
  uint32_t groups;         //!< w / 8
  uint32_t rows_per_wave;  //!< 64 / groups
  mshadow::FastDivU32 div_groups, div_h, div_c;
};

/*! \brief col2im for binary16, a 3 x 3 window, stride 1, dilation 1 and one pixel of padding
 *  (so the patch grid has the image's own height and width), w a multiple of 8, rows of
 *  whole aligned packs - the convolution-backward case - with no staging at all.
 *
 *  Every element of the column matrix belongs to exactly one pixel, and for a fixed tap
 *  (a, b) the matrix row IS an image-shaped array, shifted by (1 - a, 1 - b): the result is
 *  the sum of nine shifted streams. A thread owns 8 adjacent pixels of one image row and
 *  fetches, for each tap, the aligned pack of the tap's stream at its own place; the streams
 *  shifted by one pixel (b = 0, 2) are completed with the one missing element from the
 *  neighbouring lane, which holds the next / previous pack of the same stream (a wave takes
 *  whole rows, so the neighbour is always in the wave). Nothing is staged, no barrier: every
 *  wave is loads -> adds -> one store, and the loads of a wave are whole contiguous aligned
 *  runs of each stream.
 *
 *  The terms are added in the reference's order (py ascending = a descending, then px
 *  ascending = b descending, mshadow/extension/pack_col2patch.h:118-144) as packed binary16
 *  pairs: a binary16 add rounds after every term exactly as half_t's operator+= does. */
__global__ void __launch_bounds__(kPatchBlock)
    Col2ImHalfRows3x3Kernel(uint16_t *img, int istride, const uint16_t *col, int cstride, PatchGeom g,
                            RowsGeom rg) {
  typedef _Float16 H2 __attribute__((ext_vector_type(2)));
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = blockIdx.x * (kPatchBlock / 64) + (threadIdx.x >> 6);
  const uint32_t row_in_wave = rg.div_groups.Div(lane);
  const uint32_t group = lane - row_in_wave * rg.groups;
  const uint32_t row = wave * rg.rows_per_wave + row_in_wave;
  const bool live = row_in_wave < rg.rows_per_wave && row < rg.total_rows;
  /* lanes that own no pixels follow a neighbour's addresses: they only ever hand their
     (unused) pack to lanes that mask it */
  const uint32_t rowc = live ? row : rg.total_rows - 1u;
  const uint32_t plane = rg.div_h.Div(rowc);
  const int y = static_cast<int>(rowc - plane * g.h);
  const uint32_t n = rg.div_c.Div(plane);
  const uint32_t ch = plane - n * g.c;
  const int x0 = static_cast<int>(group * 8u);
  /* the stream of tap (a, b) at this thread's place: row py = y + 1 - a of the patch grid */
  const uint16_t *tap0 = col + static_cast<size_t>(ch) * 9u * cstride +
                         (static_cast<size_t>(n) * g.h) * g.w + x0;
  U4 q[9];
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    const int py = min(max(y + 1 - a, 0), g.h - 1);  // clamped; an absent row is skipped below
#pragma unroll
    for (int b = 0; b < 3; ++b) {
      q[a * 3 + b] = StreamLoad16(tap0 + static_cast<size_t>(a * 3 + b) * cstride +
                                  static_cast<size_t>(py) * g.w);
    }
  }
  /* the pixel left of the row (b = 2 at x = 0) and right of it (b = 0 at x = w - 1) do not exist */
  const uint32_t keep_first = group == 0u ? 0xffff0000u : 0xffffffffu;
  const uint32_t keep_last = group + 1u == rg.groups ? 0x0000ffffu : 0xffffffffu;
  uint32_t res[4] = {0u, 0u, 0u, 0u};  // eight binary16 zeros
#define MSHADOW_COL2IM_ADD(d, term, keep)                         \
  {                                                               \
    H2 acc_, term_;                                               \
    const uint32_t t_ = (term);                                   \
    __builtin_memcpy(&acc_, &res[d], 4);                          \
    __builtin_memcpy(&term_, &t_, 4);                             \
    const H2 sum_ = acc_ + term_;                                 \
    uint32_t s_;                                                  \
    __builtin_memcpy(&s_, &sum_, 4);                              \
    res[d] = ((keep) == 0xffffffffu) ? s_ : ((s_ & (keep)) | (res[d] & ~(keep))); \
  }
#pragma unroll
  for (int a = 2; a >= 0; --a) {
    const int py = y + 1 - a;
    /* the neighbours' packs are fetched by every lane (DPP needs the whole wave) */
    const U4 c2 = q[a * 3 + 2], c1 = q[a * 3 + 1], c0 = q[a * 3 + 0];
    const uint32_t prev_last = static_cast<uint32_t>(
        __builtin_amdgcn_update_dpp(0, static_cast<int>(c2.w), 0x138, 0xf, 0xf, false));  // wave_shr:1
    const uint32_t next_first = static_cast<uint32_t>(
        __builtin_amdgcn_update_dpp(0, static_cast<int>(c0.x), 0x130, 0xf, 0xf, false));  // wave_shl:1
    if (py >= 0 && py < g.h) {
      /* b = 2: pixels x - 1 */
      MSHADOW_COL2IM_ADD(0, __builtin_amdgcn_alignbit(c2.x, prev_last, 16), keep_first)
      MSHADOW_COL2IM_ADD(1, __builtin_amdgcn_alignbit(c2.y, c2.x, 16), 0xffffffffu)
      MSHADOW_COL2IM_ADD(2, __builtin_amdgcn_alignbit(c2.z, c2.y, 16), 0xffffffffu)
      MSHADOW_COL2IM_ADD(3, __builtin_amdgcn_alignbit(c2.w, c2.z, 16), 0xffffffffu)
      /* b = 1: the pixels themselves */
      MSHADOW_COL2IM_ADD(0, c1.x, 0xffffffffu)
      MSHADOW_COL2IM_ADD(1, c1.y, 0xffffffffu)
      MSHADOW_COL2IM_ADD(2, c1.z, 0xffffffffu)
      MSHADOW_COL2IM_ADD(3, c1.w, 0xffffffffu)
      /* b = 0: pixels x + 1 */
      MSHADOW_COL2IM_ADD(0, __builtin_amdgcn_alignbit(c0.y, c0.x, 16), 0xffffffffu)
      MSHADOW_COL2IM_ADD(1, __builtin_amdgcn_alignbit(c0.z, c0.y, 16), 0xffffffffu)
      MSHADOW_COL2IM_ADD(2, __builtin_amdgcn_alignbit(c0.w, c0.z, 16), 0xffffffffu)
      MSHADOW_COL2IM_ADD(3, __builtin_amdgcn_alignbit(next_first, c0.w, 16), keep_last)
    }
  }
#undef MSHADOW_COL2IM_ADD
  if (live) {
    U4 out;
    out.x = res[0], out.y = res[1], out.z = res[2], out.w = res[3];
    StreamStore16(img + static_cast<size_t>(row) * istride + x0, out);
  }
}

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

/*! \brief the divisions by stride and dilation that col2im's patch ranges need, as multiplications */
struct PatchDivs {
  mshadow::FastDivU32 sy, sx, dy, dx;
};

/*! \brief col2im for any stride and dilation, no staging: a thread sums one pack of an image row
 *  (the last pack of a row moved back to end with the row), pixel by pixel over the patches
 *  that cover it, exactly the loops of mshadow/extension/pack_col2patch.h:118-144 with the
 *  divisions done by multiplication; the terms come by element-sized loads, which neighbouring
 *  lanes and pixels share cache lines for. For strides above 1, where a pixel has few patches. */
template <typename T>
__global__ void __launch_bounds__(kPatchBlock)
    Col2ImGatherKernel(T *img, int istride, const T *col, int cstride, PatchGeom g, PatchDivs dv,
                       mshadow::FastDivU32 div_wpk, mshadow::FastDivU32 div_h,
                       mshadow::FastDivU32 div_c, uint32_t total_packs) {
  const int EPT = 16 / sizeof(T);
  const uint32_t pk = blockIdx.x * kPatchBlock + threadIdx.x;
  if (pk >= total_packs) return;
  const uint32_t rowi = div_wpk.Div(pk);             // (n * c + ch) * h + cy
  const int x0 = min(static_cast<int>(pk - rowi * div_wpk.div) * EPT, g.w - EPT);
  const uint32_t plane = div_h.Div(rowi);
  const int cy = static_cast<int>(rowi - plane * g.h);
  const uint32_t n = div_c.Div(plane);
  const uint32_t ch = plane - n * g.c;
  const int span_y = g.dy * (g.ky - 1) + 1;
  const int span_x = g.dx * (g.kx - 1) + 1;
  const int y = cy + g.pad_y;                        // position in the padded image
  const int py_min = y < span_y ? static_cast<int>(dv.dy.Mod(y)) : static_cast<int>(dv.sy.Div(y - span_y + g.sy));
  const int py_max = min(static_cast<int>(dv.sy.Div(y + g.sy)), g.oh);
  const T *base = col + static_cast<size_t>(ch) * g.ky * g.kx * cstride + static_cast<size_t>(n) * g.oh * g.ow;
  U4 acc = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int x = x0 + e + g.pad_x;
    const int px_min = x < span_x ? static_cast<int>(dv.dx.Mod(x)) : static_cast<int>(dv.sx.Div(x - span_x + g.sx));
    const int px_max = min(static_cast<int>(dv.sx.Div(x + g.sx)), g.ow);
    T res = Acc<T>::Zero();
    for (int py = py_min; py < py_max; py += g.dy) {
      const int a = static_cast<int>(dv.dy.Div(y - py * g.sy));
      for (int px = px_min; px < px_max; px += g.dx) {
        const int b = static_cast<int>(dv.dx.Div(x - px * g.sx));
        res = Acc<T>::Add(res, base[static_cast<size_t>(a * g.kx + b) * cstride + py * g.ow + px]);
      }
    }
    SetPackElement(&acc, e, res);
  }
  StorePackAnywhere(img + static_cast<size_t>(rowi) * istride + x0, acc);
}

/*! \brief Col2ImGatherKernel for dilation 1 and at most TY x TX patches over a pixel (TY >=
 *  ceil(ky / sy), TX >= ceil(kx / sx)): the same terms in the same order, but all of a thread's
 *  loads are issued before the first add. The loops of the general kernel have bounds that
 *  differ from pixel to pixel, so its loads wait for one another, 18 round trips to memory a
 *  thread for 3x3 windows with stride 2; here the patches a pixel lacks are loaded from a valid
 *  address all the same and enter the sum as +0, which changes no bit of it (a sum that starts
 *  at +0 is never -0). */
template <typename T, int TY, int TX>
__global__ void __launch_bounds__(kPatchBlock)
    Col2ImGatherFlatKernel(T *img, int istride, const T *col, int cstride, PatchGeom g, PatchDivs dv,
                           mshadow::FastDivU32 div_wpk, mshadow::FastDivU32 div_h,
                           mshadow::FastDivU32 div_c, uint32_t total_packs) {
  const int EPT = 16 / sizeof(T);
  const uint32_t pk = blockIdx.x * kPatchBlock + threadIdx.x;
  if (pk >= total_packs) return;
  const uint32_t rowi = div_wpk.Div(pk);             // (n * c + ch) * h + cy
  const int x0 = min(static_cast<int>(pk - rowi * div_wpk.div) * EPT, g.w - EPT);
  const uint32_t plane = div_h.Div(rowi);
  const int cy = static_cast<int>(rowi - plane * g.h);
  const uint32_t n = div_c.Div(plane);
  const uint32_t ch = plane - n * g.c;
  const int y = cy + g.pad_y;                        // position in the padded image
  const int py_min = y < g.ky ? 0 : static_cast<int>(dv.sy.Div(y - g.ky + g.sy));
  const int py_max = min(static_cast<int>(dv.sy.Div(y + g.sy)), g.oh);
  const T *base = col + static_cast<size_t>(ch) * g.ky * g.kx * cstride + static_cast<size_t>(n) * g.oh * g.ow;
  T term[EPT][TY][TX];
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int x = x0 + e + g.pad_x;
    const int px_min = x < g.kx ? 0 : static_cast<int>(dv.sx.Div(x - g.kx + g.sx));
    const int px_max = min(static_cast<int>(dv.sx.Div(x + g.sx)), g.ow);
#pragma unroll
    for (int i = 0; i < TY; ++i) {
      const int py = py_min + i;
      const int a = y - py * g.sy;
#pragma unroll
      for (int j = 0; j < TX; ++j) {
        const int px = px_min + j;
        const int b = x - px * g.sx;
        const bool there = py < py_max && px < px_max;
        const size_t at = there ? static_cast<size_t>(a * g.kx + b) * cstride + py * g.ow + px : 0;
        const T v = base[at];
        term[e][i][j] = there ? v : Acc<T>::Zero();
      }
    }
  }
  U4 acc = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    T res = Acc<T>::Zero();
#pragma unroll
    for (int i = 0; i < TY; ++i) {
#pragma unroll
      for (int j = 0; j < TX; ++j) res = Acc<T>::Add(res, term[e][i][j]);
    }
    SetPackElement(&acc, e, res);
  }
  StorePackAnywhere(img + static_cast<size_t>(rowi) * istride + x0, acc);
}

/*! \brief eight bytes of the column matrix at any element border */
typedef uint64_t U64Loose __attribute__((aligned(2)));

/*! \brief element k (of sizeof(T) bytes) of eight bytes */
template <typename T>
__device__ __forceinline__ T ElementOf64(uint64_t q, int k) {
  const uint32_t w = static_cast<uint32_t>(q >> (8 * sizeof(T) * k));
  T v;
  __builtin_memcpy(&v, &w, sizeof(T));
  return v;
}

/*! \brief Col2ImGatherFlatKernel for a step of two between patches along x (sx == 2, dilation 1,
 *  ow >= 8 / sizeof(T)): the pixels of one parity among a thread's pack take, for their j-th patch,
 *  NEIGHBOURING elements of one row of the column matrix (tap column b = x - 2 * px is the same
 *  for all of them), so they come as one 8-byte load instead of one load each: a quarter (half,
 *  for floats) of the requests. A pixel's patches are counted from floor((x - kx) / 2) + 1 also
 *  where that is negative; patches left of 0 or right of ow - 1 are shifted out of the 8 bytes
 *  (the load itself is moved inside the row) and enter the sum as +0, in their place in the
 *  ascending order of px. TY >= ceil(ky / sy), TX >= ceil(kx / 2). */
template <typename T, int TY, int TX>
__global__ void __launch_bounds__(kPatchBlock)
    Col2ImGatherS2Kernel(T *img, int istride, const T *col, int cstride, PatchGeom g, PatchDivs dv,
                         mshadow::FastDivU32 div_wpk, mshadow::FastDivU32 div_h,
                         mshadow::FastDivU32 div_c, uint32_t total_packs) {
  const int EPT = 16 / sizeof(T);
  const int PAIR = EPT / 2;                // pixels of one parity
  const int EB = 8 * sizeof(T);
  const uint32_t pk = blockIdx.x * kPatchBlock + threadIdx.x;
  if (pk >= total_packs) return;
  const uint32_t rowi = div_wpk.Div(pk);             // (n * c + ch) * h + cy
  const int x0 = min(static_cast<int>(pk - rowi * div_wpk.div) * EPT, g.w - EPT);
  const uint32_t plane = div_h.Div(rowi);
  const int cy = static_cast<int>(rowi - plane * g.h);
  const uint32_t n = div_c.Div(plane);
  const uint32_t ch = plane - n * g.c;
  const int y = cy + g.pad_y;                        // position in the padded image
  const int py_min = y < g.ky ? 0 : static_cast<int>(dv.sy.Div(y - g.ky + g.sy));
  const int py_max = min(static_cast<int>(dv.sy.Div(y + g.sy)), g.oh);
  const T *base = col + static_cast<size_t>(ch) * g.ky * g.kx * cstride + static_cast<size_t>(n) * g.oh * g.ow;
  uint64_t pack[2][TY][TX];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int x = x0 + p + g.pad_x;                  // first pixel of this parity
    const int px_lo = ((x - g.kx) >> 1) + 1;         // floor((x - kx) / 2) + 1, may be negative
#pragma unroll
    for (int j = 0; j < TX; ++j) {
      const int first = px_lo + j;                   // patch of the first pixel; + k for the k-th
      const int b = x - 2 * first;                   // < kx by construction
      const int inside = min(max(first, 0), g.ow - PAIR);
      const int moved = first - inside;
      const int shift = (moved < 0 ? -moved : moved) * EB;
#pragma unroll
      for (int i = 0; i < TY; ++i) {
        const int py = py_min + i;
        const int a = y - py * g.sy;
        const bool there = py < py_max && b >= 0 && shift < 64;
        const size_t at = there ? static_cast<size_t>(a * g.kx + b) * cstride + py * g.ow + inside : 0;
        const uint64_t q = *reinterpret_cast<const U64Loose *>(base + at);
        const uint64_t r = moved < 0 ? q << (shift & 63) : q >> (shift & 63);
        pack[p][i][j] = there ? r : 0ull;
      }
    }
  }
  U4 acc = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    T res = Acc<T>::Zero();
#pragma unroll
    for (int i = 0; i < TY; ++i) {
#pragma unroll
      for (int j = 0; j < TX; ++j) res = Acc<T>::Add(res, ElementOf64<T>(pack[e & 1][i][j], e >> 1));
    }
    SetPackElement(&acc, e, res);
  }
  StorePackAnywhere(img + static_cast<size_t>(rowi) * istride + x0, acc);
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
