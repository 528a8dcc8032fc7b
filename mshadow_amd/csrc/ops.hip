/*
 * C ABI, group 3: fixed-function operations on plain (pointer, pitch, shape) arguments.
 * Each entry validates its arguments on the host (a kernel is never launched on shapes
 * it does not cover), picks the kernel variant from shape and alignment, queues it on
 * the caller's stream and reports launch errors. See include/mshadow_hip.h.
 */
#include "abi_common.h"

#include <climits>
#include <mutex>

#include <mshadow/hip/kernels/reduce.h>
#include <mshadow/hip/kernels/reduce_dma.h>

#include "patch_kernels.h"
#include "pool_kernels.h"
#include "row_kernels.h"
#include "softmax_kernels.h"

using namespace mshadow_abi;
using namespace mshadow_hipk;

namespace {

/* minimal evaluators with the Plan interface the kernel templates expect */
template <typename T>
struct RawPlan2D {
  T *p;
  int stride;
  __device__ T &REval(unsigned y, unsigned x) { return p[static_cast<size_t>(y) * stride + x]; }
  __device__ const T &Eval(unsigned y, unsigned x) const {
    return p[static_cast<size_t>(y) * stride + x];
  }
};
template <typename T>
struct RawPlan1D {
  T *p;
  __device__ T &REval(unsigned, unsigned x) { return p[x]; }
  __device__ const T &Eval(unsigned, unsigned x) const { return p[x]; }
};

inline bool Aligned16(const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

template <typename F>
int DispatchSaver(int saver, F f) {
  switch (saver) {
    case MSHADOW_HIP_SAVETO: return f(mshadow::sv::saveto());
    case MSHADOW_HIP_PLUSTO: return f(mshadow::sv::plusto());
    case MSHADOW_HIP_MINUSTO: return f(mshadow::sv::minusto());
    case MSHADOW_HIP_MULTO: return f(mshadow::sv::multo());
    case MSHADOW_HIP_DIVTO: return f(mshadow::sv::divto());
    default: return Fail(MSHADOW_HIP_ERR_ARGUMENT, "unknown saver");
  }
}
template <typename F>
int DispatchReducer(int reducer, F f) {
  switch (reducer) {
    case MSHADOW_HIP_SUM: return f(mshadow::red::sum());
    case MSHADOW_HIP_MAX: return f(mshadow::red::maximum());
    case MSHADOW_HIP_MIN: return f(mshadow::red::minimum());
    default: return Fail(MSHADOW_HIP_ERR_ARGUMENT, "unknown reducer");
  }
}

}  // namespace

namespace {
const size_t kPatchLdsBudget = 24 * 1024;  // per workgroup (col2im: every tap's patch rows of a band)
/* input rows staged per workgroup: small bands, many workgroups in different phases per CU
   ((16,64,224,224) 3x3 stride 2: 117 us against 150 us with 40 KB) */
const size_t kIm2ColLdsBudget = 16 * 1024;
/* reductions long enough to fill the LDS ring of the direct-to-LDS kernels (which hold
   a whole CU's LDS); shorter ones run the register-staged kernels, several per CU */
const int kDmaMinRows = 2048;
const long long kDmaMinPerKept = 1ll << 16;

int MakePatchGeom(PatchGeom *g, int n, int c, int h, int w, int ky, int kx, int sy, int sx,
                  int dy, int dx, int pad_y, int pad_x) {
  if (n < 0 || c < 0 || h < 0 || w < 0) return Fail(MSHADOW_HIP_ERR_ARGUMENT, "negative shape");
  if (ky < 1 || kx < 1 || sy < 1 || sx < 1 || dy < 1 || dx < 1 || pad_y < 0 || pad_x < 0) {
    return Fail(MSHADOW_HIP_ERR_ARGUMENT, "kernel, stride, dilation must be >= 1, pad >= 0");
  }
  const int hp = h + 2 * pad_y, wp = w + 2 * pad_x;
  if (hp < ky || wp < kx || hp < dy * (ky - 1) + 1 || wp < dx * (kx - 1) + 1) {
    return Fail(MSHADOW_HIP_ERR_ARGUMENT, "image shape smaller than patch size");
  }
  g->n = n; g->c = c; g->h = h; g->w = w;
  g->ky = ky; g->kx = kx; g->sy = sy; g->sx = sx; g->dy = dy; g->dx = dx;
  g->pad_y = pad_y; g->pad_x = pad_x; g->hp = hp; g->wp = wp;
  g->oh = (hp - (dy * (ky - 1) + 1)) / sy + 1;
  g->ow = (wp - (dx * (kx - 1) + 1)) / sx + 1;
  const long long rows = static_cast<long long>(ky) * kx * c;
  const long long cols = static_cast<long long>(n) * g->oh * g->ow;
  if (rows >= (1ll << 31) || cols >= (1ll << 31) ||
      static_cast<long long>(n) * c * h >= (1ll << 31) ||
      static_cast<long long>(n) * c * h * w >= (1ll << 32)) {
    return Fail(MSHADOW_HIP_ERR_ARGUMENT, "too large for 32-bit indices");
  }
  return MSHADOW_HIP_OK;
}

template <typename T>
int Im2Col(T *col, int cstride, const T *img, int istride, const PatchGeom &g, void *stream) {
  const long long rows = static_cast<long long>(g.ky) * g.kx * g.c;
  const long long cols = static_cast<long long>(g.n) * g.oh * g.ow;
  if (rows == 0 || cols == 0) return MSHADOW_HIP_OK;
  if (col == NULL || img == NULL) return Fail(MSHADOW_HIP_ERR_ARGUMENT, "im2col: NULL tensor");
  if (cstride < cols || istride < g.w) {
    return Fail(MSHADOW_HIP_ERR_ARGUMENT, "im2col: pitch smaller than the row");
  }
  const int EPT = 16 / sizeof(T);
  const bool unit_steps = g.sy == 1 && g.sx == 1 && g.dy == 1 && g.dx == 1;
  /* the binary16 3-tap kernel without staging (below) serves this case better */
  const bool three_taps_direct = unit_steps && g.kx == 3 && g.pad_x == 1 && g.ow == g.w &&
                                 g.w % EPT == 0 && istride == g.w && cstride % EPT == 0 &&
                                 Aligned16(col) && Aligned16(img) && cols < (1ll << 31);
  if (three_taps_direct) {
    const uint32_t places = static_cast<uint32_t>(cols / EPT);
    const uint32_t per_block = kPatchBlock * kIm2ColDirectPer;
    const uint32_t chunks = (places + per_block - 1) / per_block;
    const long long pieces = (static_cast<long long>(g.c) * chunks + 7) / 8 * 8;
    const long long direct_blocks = pieces * g.ky;
    if (direct_blocks < (1ll << 31)) {
      hipLaunchKernelGGL((Im2ColRow3DirectKernel<T, kIm2ColDirectPer>),
                         dim3(static_cast<unsigned>(direct_blocks)), dim3(kPatchBlock), 0,
                         AsStream(stream), col, cstride, img, g,
                         mshadow::FastDivU32(static_cast<uint32_t>(g.ow / EPT)),
                         mshadow::FastDivU32(static_cast<uint32_t>(g.oh)), chunks,
                         mshadow::FastDivU32(chunks));
      return AfterLaunch("im2col");
    }
  }
  /* 3, 5 or 7 taps a row next to one another (4 with a step of two), a step of one or two between patches, patch rows of
     a pack or more: all taps of a tap row from one fetch of the image under them (3x3 stride 2 on
     (32,256,56,56) binary16: 27 us against 41 us with a fetch per tap; 5x5 stride 1 on (32,128,28,28):
     29 against 40 us. Three taps with a step of one keep a fetch per tap: 96 against 100 us on
     (32,256,56,56) without padding) */
  if (g.dx == 1 && (g.sx == 2 || (g.sx == 1 && g.kx >= 5)) &&
      (g.kx == 3 || g.kx == 5 || g.kx == 7 || (g.kx == 4 && g.sx == 2)) && g.ow >= EPT) {
    const long long ppr = (g.ow + EPT - 1) / EPT;
    const long long places = static_cast<long long>(g.n) * g.oh * ppr;
    const uint32_t chunks = static_cast<uint32_t>((places + kPatchBlock - 1) / kPatchBlock);
    const long long pieces = (static_cast<long long>(g.c) * chunks + 7) / 8 * 8;
    const long long blocks = pieces * g.ky;
    if (places + kPatchBlock < (1ll << 31) && blocks < (1ll << 31)) {
#define IM2COL_ROW_TAPS(KX, SX)                                                                       \
  hipLaunchKernelGGL((Im2ColRowTapsKernel<T, KX, SX>), dim3(static_cast<unsigned>(blocks)),           \
                     dim3(kPatchBlock), 0, AsStream(stream), col, cstride, img, istride, g,           \
                     mshadow::FastDivU32(static_cast<uint32_t>(ppr)),                                 \
                     mshadow::FastDivU32(static_cast<uint32_t>(g.oh)), chunks,                        \
                     mshadow::FastDivU32(chunks), static_cast<uint32_t>(places))
      if (g.sx == 1) {
        if (g.kx == 5) IM2COL_ROW_TAPS(5, 1);
        else IM2COL_ROW_TAPS(7, 1);
      } else {
        if (g.kx == 3) IM2COL_ROW_TAPS(3, 2);
        else if (g.kx == 4) IM2COL_ROW_TAPS(4, 2);
        else if (g.kx == 5) IM2COL_ROW_TAPS(5, 2);
        else IM2COL_ROW_TAPS(7, 2);
      }
#undef IM2COL_ROW_TAPS
      return AfterLaunch("im2col");
    }
  }
  /* stride 1, dilation 1, patch rows of a pack or more: pack by pack, no staging */
  if (unit_steps && g.ow >= EPT) {
    const long long ppr = (g.ow + EPT - 1) / EPT;
    const long long places = static_cast<long long>(g.n) * g.oh * ppr;
    const uint32_t chunks = static_cast<uint32_t>((places + kPatchBlock - 1) / kPatchBlock);
    const long long pieces = (static_cast<long long>(g.c) * chunks + 7) / 8 * 8;
    const long long blocks = pieces * g.ky * g.kx;
    if (places + kPatchBlock < (1ll << 31) && blocks < (1ll << 31)) {
      hipLaunchKernelGGL((Im2ColDirectS1Kernel<T>), dim3(static_cast<unsigned>(blocks)),
                         dim3(kPatchBlock), 0, AsStream(stream), col, cstride, img, istride, g,
                         mshadow::FastDivU32(static_cast<uint32_t>(ppr)),
                         mshadow::FastDivU32(static_cast<uint32_t>(g.oh)), chunks,
                         mshadow::FastDivU32(chunks), static_cast<uint32_t>(places));
      return AfterLaunch("im2col");
    }
  }
  /* a step of two between patches (the usual strided convolution): the same, every pack made of
     every second element of two fetched packs (3x3 stride 2 on (32,256,56,56) binary16: 42 us
     against 64 us for the staged kernel below) */
  if (g.sx == 2 && g.ow >= EPT) {
    const long long ppr = (g.ow + EPT - 1) / EPT;
    const long long places = static_cast<long long>(g.n) * g.oh * ppr;
    const uint32_t chunks = static_cast<uint32_t>((places + kPatchBlock - 1) / kPatchBlock);
    const long long pieces = (static_cast<long long>(g.c) * chunks + 7) / 8 * 8;
    const long long blocks = pieces * g.ky * g.kx;
    if (places + kPatchBlock < (1ll << 31) && blocks < (1ll << 31)) {
      hipLaunchKernelGGL((Im2ColDirectS2Kernel<T>), dim3(static_cast<unsigned>(blocks)),
                         dim3(kPatchBlock), 0, AsStream(stream), col, cstride, img, istride, g,
                         mshadow::FastDivU32(static_cast<uint32_t>(ppr)),
                         mshadow::FastDivU32(static_cast<uint32_t>(g.oh)), chunks,
                         mshadow::FastDivU32(chunks), static_cast<uint32_t>(places));
      return AfterLaunch("im2col");
    }
  }
  /* tiled: padded input rows of a band of patch rows must fit the LDS budget */
  const size_t row_bytes = static_cast<size_t>(g.wp) * sizeof(T);
  const long long max_rows = static_cast<long long>(kIm2ColLdsBudget / row_bytes);
  const long long halo = static_cast<long long>(g.ky - 1) * g.dy + 1;
  long long band = max_rows >= halo ? (max_rows - halo) / g.sy + 1 : 0;
  if (band > g.oh) band = g.oh;
  const long long planes = static_cast<long long>(g.n) * g.c;
  while (band > 8 && planes * ((g.oh + band - 1) / band) < 1024) band = (band + 1) / 2;
  if (band >= 1) {
    const long long nb = (g.oh + band - 1) / band;
    band = (g.oh + nb - 1) / nb;
    PatchTile t;
    t.band = static_cast<int>(band);
    t.bands = static_cast<int>(nb);
    t.rows_max = static_cast<int>((band - 1) * g.sy + halo);
    t.pitch = g.wp;
    const long long blocks = planes * nb;
    if (blocks >= (1ll << 31)) return Fail(MSHADOW_HIP_ERR_ARGUMENT, "im2col: too many workgroups");
    const size_t lds = static_cast<size_t>(t.rows_max) * row_bytes;
    hipLaunchKernelGGL((Im2ColTiledKernel<T, EPT>), dim3(static_cast<unsigned>(blocks)),
                       dim3(kPatchBlock), lds, AsStream(stream), col, cstride, img, istride, g, t);
  } else {
    const unsigned chunks =
        static_cast<unsigned>((cols + kPatchBlock * EPT - 1) / (kPatchBlock * EPT));
    const long long blocks = rows * chunks;
    if (blocks >= (1ll << 31)) return Fail(MSHADOW_HIP_ERR_ARGUMENT, "im2col: too many workgroups");
    hipLaunchKernelGGL((Im2ColKernel<T, EPT>), dim3(static_cast<unsigned>(blocks)),
                       dim3(kPatchBlock), 0, AsStream(stream), col, cstride, img, istride, g,
                       chunks);
  }
  return AfterLaunch("im2col");
}

template <typename T>
int Col2Im(T *img, int istride, const T *col, int cstride, const PatchGeom &g, void *stream) {
  const long long cols = static_cast<long long>(g.n) * g.oh * g.ow;
  const long long total = static_cast<long long>(g.n) * g.c * g.h * g.w;
  if (total == 0) return MSHADOW_HIP_OK;
  if (col == NULL || img == NULL) return Fail(MSHADOW_HIP_ERR_ARGUMENT, "col2im: NULL tensor");
  if (cstride < cols || istride < g.w) {
    return Fail(MSHADOW_HIP_ERR_ARGUMENT, "col2im: pitch smaller than the row");
  }
  const int EPT = 16 / sizeof(T);
  /* the convolution-backward case on rows of whole aligned packs: nine shifted streams */
  if (sizeof(T) == 2 && g.ky == 3 && g.kx == 3 && g.sy == 1 && g.sx == 1 && g.dy == 1 && g.dx == 1 &&
      g.pad_y == 1 && g.pad_x == 1 && g.w % 8 == 0 && g.w <= 512 && istride % 8 == 0 &&
      cstride % 8 == 0 && Aligned16(img) && Aligned16(col) && total < (1ll << 31) &&
      static_cast<long long>(g.c) * 9 * cstride < (1ll << 40)) {
    RowsGeom rg;
    rg.total_rows = static_cast<uint32_t>(static_cast<long long>(g.n) * g.c * g.h);
    rg.groups = static_cast<uint32_t>(g.w / 8);
    rg.rows_per_wave = 64u / rg.groups;
    rg.div_groups = mshadow::FastDivU32(rg.groups);
    rg.div_h = mshadow::FastDivU32(static_cast<uint32_t>(g.h));
    rg.div_c = mshadow::FastDivU32(static_cast<uint32_t>(g.c));
    const uint32_t waves = (rg.total_rows + rg.rows_per_wave - 1) / rg.rows_per_wave;
    const uint32_t blocks = (waves + kPatchBlock / 64 - 1) / (kPatchBlock / 64);
    hipLaunchKernelGGL(Col2ImHalfRows3x3Kernel, dim3(blocks), dim3(kPatchBlock), 0, AsStream(stream),
                       reinterpret_cast<uint16_t *>(img), istride,
                       reinterpret_cast<const uint16_t *>(col), cstride, g, rg);
    return AfterLaunch("col2im");
  }
  /* stride 1, dilation 1, image rows of a pack or more: pack by pack, no staging */
  if (g.sy == 1 && g.sx == 1 && g.dy == 1 && g.dx == 1 && g.w >= EPT) {
    const long long wpk = (g.w + EPT - 1) / EPT;
    const long long packs = static_cast<long long>(g.n) * g.c * g.h * wpk;
    if (packs + kPatchBlock < (1ll << 31) && cols < (1ll << 31)) {
      const unsigned blocks = static_cast<unsigned>((packs + kPatchBlock - 1) / kPatchBlock);
      hipLaunchKernelGGL((Col2ImDirectS1Kernel<T>), dim3(blocks), dim3(kPatchBlock), 0, AsStream(stream),
                         img, istride, col, cstride, g, mshadow::FastDivU32(static_cast<uint32_t>(wpk)),
                         mshadow::FastDivU32(static_cast<uint32_t>(g.h)),
                         mshadow::FastDivU32(static_cast<uint32_t>(g.c)), static_cast<uint32_t>(packs));
      return AfterLaunch("col2im");
    }
  }
  /* strides above 1, image rows of a pack or more: a pixel has few patches, gathered directly */
  if ((g.sy > 1 || g.sx > 1) && g.w >= EPT) {
    const long long wpk = (g.w + EPT - 1) / EPT;
    const long long packs = static_cast<long long>(g.n) * g.c * g.h * wpk;
    if (packs + kPatchBlock < (1ll << 31) && cols < (1ll << 31)) {
      const unsigned blocks = static_cast<unsigned>((packs + kPatchBlock - 1) / kPatchBlock);
      const PatchDivs dv = {mshadow::FastDivU32(static_cast<uint32_t>(g.sy)),
                            mshadow::FastDivU32(static_cast<uint32_t>(g.sx)),
                            mshadow::FastDivU32(static_cast<uint32_t>(g.dy)),
                            mshadow::FastDivU32(static_cast<uint32_t>(g.dx))};
      /* dilation 1 and few patches over a pixel: every load of a thread under way at once */
      const int over_y = (g.ky + g.sy - 1) / g.sy, over_x = (g.kx + g.sx - 1) / g.sx;
      const int over = over_y > over_x ? over_y : over_x;
      if (g.dy == 1 && g.dx == 1 && over <= 4) {
#define COL2IM_FLAT(TY, TX)                                                                                  \
  hipLaunchKernelGGL((Col2ImGatherFlatKernel<T, TY, TX>), dim3(blocks), dim3(kPatchBlock), 0, AsStream(stream), \
                     img, istride, col, cstride, g, dv, mshadow::FastDivU32(static_cast<uint32_t>(wpk)),       \
                     mshadow::FastDivU32(static_cast<uint32_t>(g.h)),                                          \
                     mshadow::FastDivU32(static_cast<uint32_t>(g.c)), static_cast<uint32_t>(packs))
        /* a step of two along x: the patches of every second pixel are neighbours in the matrix */
        if (g.sx == 2 && g.ow >= EPT / 2 && over >= 2) {
#define COL2IM_S2(TY, TX)                                                                                    \
  hipLaunchKernelGGL((Col2ImGatherS2Kernel<T, TY, TX>), dim3(blocks), dim3(kPatchBlock), 0, AsStream(stream), \
                     img, istride, col, cstride, g, dv, mshadow::FastDivU32(static_cast<uint32_t>(wpk)),       \
                     mshadow::FastDivU32(static_cast<uint32_t>(g.h)),                                          \
                     mshadow::FastDivU32(static_cast<uint32_t>(g.c)), static_cast<uint32_t>(packs))
          if (over == 2) COL2IM_S2(2, 2);
          else if (over == 3) COL2IM_S2(3, 3);
          else COL2IM_S2(4, 4);
#undef COL2IM_S2
          return AfterLaunch("col2im");
        }
        if (over <= 1) COL2IM_FLAT(1, 1);
        else if (over == 2) COL2IM_FLAT(2, 2);
        else if (over == 3) COL2IM_FLAT(3, 3);
        else COL2IM_FLAT(4, 4);
#undef COL2IM_FLAT
        return AfterLaunch("col2im");
      }
      hipLaunchKernelGGL((Col2ImGatherKernel<T>), dim3(blocks), dim3(kPatchBlock), 0, AsStream(stream),
                         img, istride, col, cstride, g, dv, mshadow::FastDivU32(static_cast<uint32_t>(wpk)),
                         mshadow::FastDivU32(static_cast<uint32_t>(g.h)),
                         mshadow::FastDivU32(static_cast<uint32_t>(g.c)), static_cast<uint32_t>(packs));
      return AfterLaunch("col2im");
    }
  }
  /* tiled: per tap, the patch rows a band of image rows touches; all taps must fit */
  const long long taps = static_cast<long long>(g.ky) * g.kx;
  const size_t prow_bytes = static_cast<size_t>(taps) * g.ow * sizeof(T);
  const long long max_prows = static_cast<long long>(kPatchLdsBudget / prow_bytes);
  /* an image band of b rows touches at most (b + span_y - 2) / sy + 2 patch rows */
  const long long span_y = static_cast<long long>(g.dy) * (g.ky - 1) + 1;
  long long band = (max_prows - 2) * g.sy - span_y + 2;
  if (band > g.h) band = g.h;
  const long long planes = static_cast<long long>(g.n) * g.c;
  while (band > 8 && planes * ((g.h + band - 1) / band) < 1024) band = (band + 1) / 2;
  if (band >= 1 && max_prows >= 3) {
    const long long nb = (g.h + band - 1) / band;
    band = (g.h + nb - 1) / nb;
    PatchTile t;
    t.band = static_cast<int>(band);
    t.bands = static_cast<int>(nb);
    t.rows_max = static_cast<int>((band + span_y - 2) / g.sy + 2);
    t.pitch = (t.rows_max * g.ow + EPT - 1) / EPT * EPT;
    const size_t lds = static_cast<size_t>(taps) * t.pitch * sizeof(T);
    const long long blocks = planes * nb;
    if (blocks >= (1ll << 31)) return Fail(MSHADOW_HIP_ERR_ARGUMENT, "col2im: too many workgroups");
    if (g.dy == 1 && g.dx == 1 && g.sy == 1 && g.sx == 1) {
      hipLaunchKernelGGL((Col2ImTiledKernel<T, EPT, true>), dim3(static_cast<unsigned>(blocks)),
                         dim3(kPatchBlock), lds, AsStream(stream), img, istride, col, cstride, g, t);
    } else {
      hipLaunchKernelGGL((Col2ImTiledKernel<T, EPT, false>), dim3(static_cast<unsigned>(blocks)),
                         dim3(kPatchBlock), lds, AsStream(stream), img, istride, col, cstride, g, t);
    }
  } else {
    unsigned grid = 0;
    int st = mshadow_hip_suggest_grid(static_cast<size_t>(total), kPatchBlock, 8, &grid);
    if (st != MSHADOW_HIP_OK) return st;
    hipLaunchKernelGGL((Col2ImKernel<T>), dim3(grid), dim3(kPatchBlock), 0, AsStream(stream), img,
                       istride, col, cstride, g, static_cast<unsigned>(total));
  }
  return AfterLaunch("col2im");
}
struct UnpoolArgs {
  float *dst; int dstride; const float *src; int sstride; const float *pooled; int pstride;
  const float *grad; int gstride; PoolGeom g; int prow_max; unsigned blocks; size_t lds;
  hipStream_t s;
};
#define UNPOOL_ARGS(a) a.dst, a.dstride, a.src, a.sstride, a.pooled, a.pstride, a.grad, a.gstride, a.g, a.prow_max
template <int KY, int KX, int SY, int SX, bool VEC>
void LaunchUnpoolBlock(int reducer, const UnpoolArgs &a, const mshadow::FastDivU32 &div_bw) {
  switch (reducer) {
    case MSHADOW_HIP_SUM:
      hipLaunchKernelGGL((UnpoolBlockKernel<MSHADOW_HIP_SUM, KY, KX, SY, SX, VEC>), dim3(a.blocks),
                         dim3(kPoolBlock), a.lds, a.s, UNPOOL_ARGS(a), div_bw);
      break;
    case MSHADOW_HIP_MAX:
      hipLaunchKernelGGL((UnpoolBlockKernel<MSHADOW_HIP_MAX, KY, KX, SY, SX, VEC>), dim3(a.blocks),
                         dim3(kPoolBlock), a.lds, a.s, UNPOOL_ARGS(a), div_bw);
      break;
    default:
      hipLaunchKernelGGL((UnpoolBlockKernel<MSHADOW_HIP_MIN, KY, KX, SY, SX, VEC>), dim3(a.blocks),
                         dim3(kPoolBlock), a.lds, a.s, UNPOOL_ARGS(a), div_bw);
      break;
  }
}
void LaunchUnpoolGeneric(int reducer, const UnpoolArgs &a) {
  switch (reducer) {
    case MSHADOW_HIP_SUM:
      hipLaunchKernelGGL((UnpoolKernel<MSHADOW_HIP_SUM, 0, 0, 0, 0>), dim3(a.blocks), dim3(kPoolBlock),
                         a.lds, a.s, UNPOOL_ARGS(a));
      break;
    case MSHADOW_HIP_MAX:
      hipLaunchKernelGGL((UnpoolKernel<MSHADOW_HIP_MAX, 0, 0, 0, 0>), dim3(a.blocks), dim3(kPoolBlock),
                         a.lds, a.s, UNPOOL_ARGS(a));
      break;
    default:
      hipLaunchKernelGGL((UnpoolKernel<MSHADOW_HIP_MIN, 0, 0, 0, 0>), dim3(a.blocks), dim3(kPoolBlock),
                         a.lds, a.s, UNPOOL_ARGS(a));
      break;
  }
}
#undef UNPOOL_ARGS


struct GradLaunch {
  float *dst; int dstride; const float *src; int sstride; const float *label; int cols;
  unsigned chunks; GradParams gp; unsigned blocks; hipStream_t s;
};
template <bool VEC>
void LaunchGrad(int flags, const GradLaunch &g) {
#define GRAD2D(FLAGS)                                                                         \
  hipLaunchKernelGGL((SoftmaxGradKernel<VEC, FLAGS>), dim3(g.blocks), dim3(kGradBlock), 0, g.s, \
                     g.dst, g.dstride, g.src, g.sstride, g.label, g.cols, g.chunks, g.gp)
  switch (flags) {
    case 0: GRAD2D(0); break;
    case 1: GRAD2D(1); break;
    case 2: GRAD2D(2); break;
    default: GRAD2D(3); break;
  }
#undef GRAD2D
}


}  // namespace


template <int OP>
static int LaunchRowsByIndex(float *dst, int dstride, int k_rows, const void *rows_of,
                             const void *from_of, int index_is_int, int n_index, const float *src,
                             int sstride, int cols, void *stream, const char *what) {
  unsigned grid = 0;
  int rows_per_wave = 0;
  mshadow::hip::RowsByIndexGrid(k_rows, &grid, &rows_per_wave);
  const bool vec = Aligned16(dst) && Aligned16(src) && dstride % 4 == 0 && sstride % 4 == 0 &&
                   cols % 4 == 0;
  hipStream_t s = AsStream(stream);
#define ROWS_LAUNCH(ITYPE, VEC)                                                               \
  hipLaunchKernelGGL((RowsByIndexKernel<ITYPE, float, OP, VEC>), dim3(grid), dim3(kTakeBlock), 0, \
                     s, dst, dstride, k_rows, rows_per_wave, static_cast<const ITYPE *>(rows_of), \
                     static_cast<const ITYPE *>(from_of), n_index, src, sstride, cols)
  if (index_is_int) {
    if (vec) ROWS_LAUNCH(int32_t, true); else ROWS_LAUNCH(int32_t, false);
  } else {
    if (vec) ROWS_LAUNCH(float, true); else ROWS_LAUNCH(float, false);
  }
#undef ROWS_LAUNCH
  return AfterLaunch(what);
}

namespace {
/*! \brief rows of at most 256 columns: one thread per row up to 32 columns, one wave per row
 *  above (1, 2 or 4 columns per lane) */
template <bool TERMS_GIVEN>
void LaunchShortSoftmax(float *dst, int dstride, const float *src, int sstride, int rows, int cols,
                        hipStream_t s) {
  if (cols <= 32) {
    hipLaunchKernelGGL((SoftmaxThreadRowKernel<32, TERMS_GIVEN>), dim3((rows + 255) / 256), dim3(256),
                       0, s, dst, dstride, src, sstride, rows, cols);
  } else if (cols <= 64) {   // four rows to a wave
    hipLaunchKernelGGL((SoftmaxPartWaveKernel<16, 4, TERMS_GIVEN>), dim3((rows + 15) / 16), dim3(256), 0, s,
                       dst, dstride, src, sstride, rows, cols);
  } else if (cols <= 128) {
    hipLaunchKernelGGL((SoftmaxPartWaveKernel<16, 8, TERMS_GIVEN>), dim3((rows + 15) / 16), dim3(256), 0, s,
                       dst, dstride, src, sstride, rows, cols);
  } else {                   // two rows to a wave
    hipLaunchKernelGGL((SoftmaxPartWaveKernel<32, 8, TERMS_GIVEN>), dim3((rows + 7) / 8), dim3(256), 0, s,
                       dst, dstride, src, sstride, rows, cols);
  }
}
}  // namespace

/* Scratch memory of the split KeepHighDim reduction (kernels/reduce_dma.h): the inner results of
   a launch and the counter that tells the last workgroup. It is part of the library's image
   - a file-scope device array, one copy per GPU, nothing is allocated at run time - and is
   handed out per stream: launches on one stream run one after the other, so a stream's slot is
   never in use twice; a ninth stream on one GPU, or a launch with more inner results than a
   slot holds, gets none and its reduction runs the one-workgroup-per-kept-index kernel. */
namespace {
const int kReduceScratchSlots = 8;
const size_t kReduceScratchWords = 1u << 16;
const int kReduceScratchDevices = 16;
struct ReduceScratchSlot {
  uint32_t partial[kReduceScratchWords];
  uint32_t counter[mshadow::hip::kSplitCounterWords];  // zero between launches
};
static __device__ __align__(256) ReduceScratchSlot g_reduce_scratch[kReduceScratchSlots];

struct ReduceScratchTable {
  std::mutex mu;
  ReduceScratchSlot *base[kReduceScratchDevices];
  bool used[kReduceScratchDevices][kReduceScratchSlots];
  void *owner[kReduceScratchDevices][kReduceScratchSlots];
};
ReduceScratchTable &ScratchTable() {
  static ReduceScratchTable t = {};
  return t;
}
}  // namespace

namespace mshadow_abi {
void ReleaseReduceScratch(void *stream) {
  ReduceScratchTable &t = ScratchTable();
  std::lock_guard<std::mutex> lock(t.mu);
  for (int d = 0; d < kReduceScratchDevices; ++d) {
    for (int i = 0; i < kReduceScratchSlots; ++i) {
      if (t.used[d][i] && t.owner[d][i] == stream) t.used[d][i] = false;
    }
  }
}
/* called when a device is selected: where the scratch array lives on that device is looked up
   then, not inside the first reduction that wants a slot (which may be being recorded) */
void ResolveReduceScratch() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kReduceScratchDevices) {
    (void)hipGetLastError();
    return;
  }
  ReduceScratchTable &t = ScratchTable();
  std::lock_guard<std::mutex> lock(t.mu);
  if (t.base[dev] == NULL) {
    void *p = NULL;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_reduce_scratch)) == hipSuccess) {
      t.base[dev] = static_cast<ReduceScratchSlot *>(p);
    } else {
      (void)hipGetLastError();
    }
  }
}
}  // namespace mshadow_abi

extern "C" int mshadow_hip_reduce_scratch(void *stream, size_t words, uint32_t **partial,
                                          uint32_t **counter) {
  ABI_REQUIRE(partial != NULL && counter != NULL, "NULL result");
  *partial = NULL;
  *counter = NULL;
  if (words > kReduceScratchWords) return MSHADOW_HIP_OK;
  int dev = 0;
  ABI_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kReduceScratchDevices) return MSHADOW_HIP_OK;
  ReduceScratchTable &t = ScratchTable();
  std::lock_guard<std::mutex> lock(t.mu);
  if (t.base[dev] == NULL) {
    /* the array's name is a host-side stand-in; this is its address on the current device */
    void *p = NULL;
    ABI_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_reduce_scratch)));
    t.base[dev] = static_cast<ReduceScratchSlot *>(p);
  }
  int slot = -1;
  for (int i = 0; i < kReduceScratchSlots && slot < 0; ++i) {
    if (t.used[dev][i] && t.owner[dev][i] == stream) slot = i;
  }
  for (int i = 0; i < kReduceScratchSlots && slot < 0; ++i) {
    if (!t.used[dev][i]) {
      t.used[dev][i] = true;
      t.owner[dev][i] = stream;
      slot = i;
    }
  }
  if (slot < 0) return MSHADOW_HIP_OK;
  *partial = t.base[dev][slot].partial;
  *counter = t.base[dev][slot].counter;
  return MSHADOW_HIP_OK;
}

extern "C" {

/* ------------------------------------------------------------------ softmax */

int mshadow_hip_softmax_f32(float *dst, int dstride, const float *src, int sstride, int rows,
                            int cols, void *stream) {
  ABI_REQUIRE(rows >= 0 && cols >= 0, "negative shape");
  if (rows == 0 || cols == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL && src != NULL, "NULL tensor");
  ABI_REQUIRE(dstride >= cols && sstride >= cols, "pitch smaller than the row");
  hipStream_t s = AsStream(stream);
  if (cols <= 256) {  // short rows: a thread or a wave per row instead of a workgroup
    LaunchShortSoftmax<false>(dst, dstride, src, sstride, rows, cols, s);
    return AfterLaunch("softmax");
  }
  /* 16-byte packs wherever the rows start and whatever their length (the accesses need no
     alignment; a row's last, partial pack goes element by element) */
#define SOFTMAX_LAUNCH(T, S, V) \
  hipLaunchKernelGGL((SoftmaxRowKernel<T, S, V, false>), dim3(rows), dim3(T), 0, s, dst, dstride, \
                     src, sstride, cols)
#define SOFTMAX_WAVE(SLABS) \
  hipLaunchKernelGGL((SoftmaxWaveSlabsKernel<SLABS, false>), dim3((rows + 3) / 4), dim3(256), 0, s, dst, \
                     dstride, src, sstride, rows, cols)
  /* many rows of up to 3072 columns: a wave per row (65536 rows of 300 / 1000 / 2000 columns:
     71 / 109 / 122 us against 163 / 193 / 139 us with a workgroup per row; 16384 rows of 2304 /
     3000 columns: 80 / 98 us against 120 / 133 us; at 4096 columns, 64 of them a lane, the wave
     takes 176 us against 127 us, and with few rows the workgroup per row is faster) */
  if (cols <= 3072 && rows >= 8 * mshadow_abi::ComputeUnits()) {
    if (cols <= 512) SOFTMAX_WAVE(2);
    else if (cols <= 1024) SOFTMAX_WAVE(4);
    else if (cols <= 2048) SOFTMAX_WAVE(8);
    else SOFTMAX_WAVE(12);
    return AfterLaunch("softmax");
  }
  /* many rows of 8193 to 16384 columns: four waves a row with 64 columns a thread, eight rows to a
     CU instead of four ((4096,10000): 82 against 104 us, (8192,12288): 153 against 196 us; with
     2048 rows the eight waves a row below finish them sooner, 57 against 70 us) */
  if (cols > 8192 && cols <= 16384 && rows >= 16 * mshadow_abi::ComputeUnits()) {
    SOFTMAX_LAUNCH(256, 16, 4);
    return AfterLaunch("softmax");
  }
#undef SOFTMAX_WAVE
  if (cols <= 1024) SOFTMAX_LAUNCH(256, 1, 4);
  else if (cols <= 2048) SOFTMAX_LAUNCH(256, 2, 4);
  else if (cols <= 4096) SOFTMAX_LAUNCH(256, 4, 4);
  else if (cols <= 8192) SOFTMAX_LAUNCH(256, 8, 4);
  else if (cols <= 16384) SOFTMAX_LAUNCH(512, 8, 4);
  else if (cols <= 32768) SOFTMAX_LAUNCH(512, 16, 4);
  else if (cols <= 65536) SOFTMAX_LAUNCH(1024, 16, 4);
  /* longer rows: stretches of 32768 columns on 512 threads, two rows to a CU ((512,128000): 221 us
     against 271 us with stretches of 65536 on 1024 threads; up to 65536 columns the single pass
     above is faster than stretches, 265 against 432 us on (2048,50257)) */
  else if (cols > INT_MAX - 32768) {
    return Fail(MSHADOW_HIP_ERR_ARGUMENT, "softmax: row too long for 32-bit column counts");
  } else if (rows > mshadow_abi::ComputeUnits()) {
    hipLaunchKernelGGL((SoftmaxStretchRowKernel<512, 16, false, 4>), dim3(rows), dim3(512), 0, s, dst,
                       dstride, src, sstride, cols);
  } else {
    hipLaunchKernelGGL((SoftmaxStretchRowKernel<512, 16, false, 2>), dim3(rows), dim3(512), 0, s, dst,
                       dstride, src, sstride, cols);
  }
#undef SOFTMAX_LAUNCH
  return AfterLaunch("softmax");
}

int mshadow_hip_softmax_rowsum_f32(float *sums, const float *terms, int tstride, int rows,
                                   int cols, void *stream) {
  ABI_REQUIRE(rows >= 0 && cols >= 0, "negative shape");
  if (rows == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(sums != NULL && (terms != NULL || cols == 0), "NULL tensor");
  ABI_REQUIRE(tstride >= cols, "pitch smaller than the row");
  hipStream_t s = AsStream(stream);
  if (cols <= 256) {
    LaunchShortSoftmax<true>(sums, 0, terms, tstride, rows, cols, s);
    return AfterLaunch("softmax_rowsum");
  }
  if (cols <= 3072 && rows >= 8 * mshadow_abi::ComputeUnits()) {  // as in mshadow_hip_softmax_f32
#define ROWSUM_WAVE(SLABS) \
  hipLaunchKernelGGL((SoftmaxWaveSlabsKernel<SLABS, true>), dim3((rows + 3) / 4), dim3(256), 0, s, sums, 0, \
                     terms, tstride, rows, cols)
    if (cols <= 512) ROWSUM_WAVE(2);
    else if (cols <= 1024) ROWSUM_WAVE(4);
    else if (cols <= 2048) ROWSUM_WAVE(8);
    else ROWSUM_WAVE(12);
#undef ROWSUM_WAVE
    return AfterLaunch("softmax_rowsum");
  }
  const bool vec = Aligned16(terms) && tstride % 4 == 0 && cols % 4 == 0;
  /* rows longer than a workgroup's registers hold: stretch by stretch, at any alignment */
  if (cols > 65536 || (!vec && cols > 32768)) {
    ABI_REQUIRE(cols <= INT_MAX - 32768, "row too long for 32-bit column counts");
    hipLaunchKernelGGL((SoftmaxStretchRowKernel<512, 16, true, 2>), dim3(rows), dim3(512), 0, s, sums, 0,
                       terms, tstride, cols);
    return AfterLaunch("softmax_rowsum");
  }
#define ROWSUM_LAUNCH(T, S, V) \
  hipLaunchKernelGGL((SoftmaxRowKernel<T, S, V, true>), dim3(rows), dim3(T), 0, s, sums, 0, terms, \
                     tstride, cols)
  if (vec) {
    if (cols > 8192 && cols <= 16384 && rows >= 16 * mshadow_abi::ComputeUnits()) ROWSUM_LAUNCH(256, 16, 4);  // as above
    else if (cols <= 1024) ROWSUM_LAUNCH(256, 1, 4);
    else if (cols <= 2048) ROWSUM_LAUNCH(256, 2, 4);
    else if (cols <= 4096) ROWSUM_LAUNCH(256, 4, 4);
    else if (cols <= 8192) ROWSUM_LAUNCH(256, 8, 4);
    else if (cols <= 16384) ROWSUM_LAUNCH(512, 8, 4);
    else if (cols <= 32768) ROWSUM_LAUNCH(512, 16, 4);
    else ROWSUM_LAUNCH(1024, 16, 4);
  } else {
    if (cols <= 1024) ROWSUM_LAUNCH(256, 4, 1);
    else if (cols <= 4096) ROWSUM_LAUNCH(256, 16, 1);
    else if (cols <= 16384) ROWSUM_LAUNCH(1024, 16, 1);
    else ROWSUM_LAUNCH(1024, 32, 1);
  }
#undef ROWSUM_LAUNCH
  return AfterLaunch("softmax_rowsum");
}

int mshadow_hip_softmax_grad_ex_f32(float *dst, int dstride, const float *src, int sstride,
                                    const float *label, int rows, int cols, int flags,
                                    float ignore_label, float alpha, void *stream) {
  ABI_REQUIRE(rows >= 0 && cols >= 0, "negative shape");
  ABI_REQUIRE(flags >= 0 && flags <= 3, "unknown gradient flags");
  if (rows == 0 || cols == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL && src != NULL && label != NULL, "NULL tensor");
  ABI_REQUIRE(dstride >= cols && sstride >= cols, "pitch smaller than the row");
  const int per_block = kGradBlock * kGradPacks * 4;
  const unsigned chunks = (cols + per_block - 1) / per_block;
  const unsigned long long blocks = static_cast<unsigned long long>(rows) * chunks;
  ABI_REQUIRE(blocks < (1ull << 31), "too many workgroups");
  /* alpha / (classes - 1) with the count converted from unsigned, as the reference writes it */
  const GradParams gp = {static_cast<int>(ignore_label), alpha,
                         alpha / static_cast<float>(static_cast<unsigned>(cols - 1))};
  if (cols <= 512) {  // short rows: several to a workgroup, a pack a thread
    const int ppr = (cols + 3) / 4;
    const int rows_per_block = kGradBlock / ppr;
    const unsigned grid = static_cast<unsigned>((rows + rows_per_block - 1) / rows_per_block);
    const mshadow::FastDivU32 div_ppr(static_cast<uint32_t>(ppr));
#define GRAD_SHORT(FLAGS)                                                                            \
  hipLaunchKernelGGL((SoftmaxGradShortRowsKernel<FLAGS>), dim3(grid), dim3(kGradBlock), 0, AsStream(stream), \
                     dst, dstride, src, sstride, label, rows, cols, rows_per_block, div_ppr, gp)
    switch (flags) {
      case 0: GRAD_SHORT(0); break;
      case 1: GRAD_SHORT(1); break;
      case 2: GRAD_SHORT(2); break;
      default: GRAD_SHORT(3); break;
    }
#undef GRAD_SHORT
    return AfterLaunch("softmax_grad");
  }
  GradLaunch gl = {dst, dstride, src, sstride, label, cols, chunks, gp,
                   static_cast<unsigned>(blocks), AsStream(stream)};
  LaunchGrad<true>(flags, gl);   // 16-byte packs wherever the rows start (no alignment needed)
  return AfterLaunch("softmax_grad");
}

int mshadow_hip_softmax_grad_f32(float *dst, int dstride, const float *src, int sstride,
                                 const float *label, int rows, int cols, void *stream) {
  return mshadow_hip_softmax_grad_ex_f32(dst, dstride, src, sstride, label, rows, cols, 0, 0.0f,
                                         0.0f, stream);
}

int mshadow_hip_softmax3d_f32(float *dst, int dstride, const float *src, int sstride, int d0,
                              int d1, int d2, void *stream) {
  ABI_REQUIRE(d0 >= 0 && d1 >= 0 && d2 >= 0, "negative shape");
  if (d0 == 0 || d1 == 0 || d2 == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL && src != NULL, "NULL tensor");
  ABI_REQUIRE(dstride >= d2 && sstride >= d2, "pitch smaller than the row");
  ABI_REQUIRE(static_cast<long long>(d0) * d2 < (1ll << 31) &&
                  static_cast<long long>(d0) * d1 < (1ll << 31),
              "too large for 32-bit indices");
  const mshadow::FastDivU32 div_d2s(static_cast<uint32_t>(d2));
  const unsigned pairs = static_cast<unsigned>(d0) * d2;
  const unsigned one_each = (pairs + kSoftmax3dBlock - 1) / kSoftmax3dBlock;
  if (d1 <= 8) {
    hipLaunchKernelGGL((Softmax3dSmallKernel<8>), dim3(one_each), dim3(kSoftmax3dBlock), 0,
                       AsStream(stream), dst, dstride, src, sstride, d0, d1, d2, div_d2s);
    return AfterLaunch("softmax3d");
  }
  if (d1 <= 32) {
    hipLaunchKernelGGL((Softmax3dSmallKernel<32>), dim3(one_each), dim3(kSoftmax3dBlock), 0,
                       AsStream(stream), dst, dstride, src, sstride, d0, d1, d2, div_d2s);
    return AfterLaunch("softmax3d");
  }
  unsigned grid = 0;
  int st = mshadow_hip_suggest_grid(static_cast<size_t>(d0) * d2, kSoftmax3dBlock, 8, &grid);
  if (st != MSHADOW_HIP_OK) return st;
  hipLaunchKernelGGL(Softmax3dKernel, dim3(grid), dim3(kSoftmax3dBlock), 0, AsStream(stream), dst,
                     dstride, src, sstride, d0, d1, d2,
                     mshadow::FastDivU32(static_cast<uint32_t>(d2)));
  return AfterLaunch("softmax3d");
}

int mshadow_hip_softmax3d_grad_f32(float *dst, int dstride, const float *src, int sstride,
                                   const float *label, int lstride, int d0, int d1, int d2,
                                   int flags, float ignore_label, float alpha, void *stream) {
  ABI_REQUIRE(d0 >= 0 && d1 >= 0 && d2 >= 0, "negative shape");
  ABI_REQUIRE(flags >= 0 && flags <= 3, "unknown gradient flags");
  if (d0 == 0 || d1 == 0 || d2 == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL && src != NULL && label != NULL, "NULL tensor");
  ABI_REQUIRE(dstride >= d2 && sstride >= d2 && lstride >= d2, "pitch smaller than the row");
  ABI_REQUIRE(static_cast<long long>(d0) * d1 * d2 < (1ll << 31), "too large for 32-bit indices");
  unsigned grid = 0;
  int st = mshadow_hip_suggest_grid(static_cast<size_t>(d0) * d1 * d2, kSoftmax3dBlock, 8, &grid);
  if (st != MSHADOW_HIP_OK) return st;
  const GradParams gp = {static_cast<int>(ignore_label), alpha,
                         alpha / static_cast<float>(static_cast<unsigned>(d1 - 1))};
  const mshadow::FastDivU32 div_d2(static_cast<uint32_t>(d2)), div_d1(static_cast<uint32_t>(d1));
  const bool vec = d2 % 4 == 0 && dstride % 4 == 0 && sstride % 4 == 0 && lstride % 4 == 0 &&
                   Aligned16(dst) && Aligned16(src) && Aligned16(label);
  if (vec) {
    const unsigned packs = static_cast<unsigned>(d0) * d1 * (d2 / 4);
    const unsigned vgrid = (packs + kSoftmax3dBlock - 1) / kSoftmax3dBlock;
    const mshadow::FastDivU32 div_q2(static_cast<uint32_t>(d2 / 4));
#define GRAD3DV(FLAGS)                                                                         \
  hipLaunchKernelGGL((Softmax3dGradVecKernel<FLAGS>), dim3(vgrid), dim3(kSoftmax3dBlock), 0,   \
                     AsStream(stream), dst, dstride, src, sstride, label, lstride, d0, d1, d2, \
                     div_q2, div_d1, gp)
    switch (flags) {
      case 0: GRAD3DV(0); break;
      case 1: GRAD3DV(1); break;
      case 2: GRAD3DV(2); break;
      default: GRAD3DV(3); break;
    }
#undef GRAD3DV
    return AfterLaunch("softmax3d_grad");
  }
#define GRAD3D(FLAGS)                                                                          \
  hipLaunchKernelGGL((Softmax3dGradKernel<FLAGS>), dim3(grid), dim3(kSoftmax3dBlock), 0,       \
                     AsStream(stream), dst, dstride, src, sstride, label, lstride, d0, d1, d2, \
                     div_d2, div_d1, gp)
  switch (flags) {
    case 0: GRAD3D(0); break;
    case 1: GRAD3D(1); break;
    case 2: GRAD3D(2); break;
    default: GRAD3D(3); break;
  }
#undef GRAD3D
  return AfterLaunch("softmax3d_grad");
}

static int RowOpCheck(const float *dst, int dstride, int k_rows, const void *index, int n_index,
                      const float *src, int sstride, int cols) {
  ABI_REQUIRE(k_rows >= 0 && n_index >= 0 && cols >= 0, "negative shape");
  if (k_rows == 0 || n_index == 0 || cols == 0) return -1;  // nothing to do
  ABI_REQUIRE(dst != NULL && src != NULL && index != NULL, "NULL tensor");
  ABI_REQUIRE(dstride >= cols && sstride >= cols, "pitch smaller than the row");
  return MSHADOW_HIP_OK;
}

int mshadow_hip_add_take_grad_f32(float *dst, int dstride, int k_rows, const void *index,
                                  int index_is_int, int n_index, const float *src, int sstride,
                                  int cols, void *stream) {
  const int chk = RowOpCheck(dst, dstride, k_rows, index, n_index, src, sstride, cols);
  if (chk != MSHADOW_HIP_OK) return chk < 0 ? MSHADOW_HIP_OK : chk;
  return LaunchRowsByIndex<kTakeGrad>(dst, dstride, k_rows, index, index, index_is_int, n_index,
                                      src, sstride, cols, stream, "add_take_grad");
}

int mshadow_hip_add_take_grad_large_batch_f32(float *dst, int dstride, int k_rows,
                                              const void *sorted, const void *index,
                                              int index_is_int, int n_index, const float *src,
                                              int sstride, int cols, void *stream) {
  const int chk = RowOpCheck(dst, dstride, k_rows, index, n_index, src, sstride, cols);
  if (chk != MSHADOW_HIP_OK) return chk < 0 ? MSHADOW_HIP_OK : chk;
  ABI_REQUIRE(sorted != NULL, "NULL tensor");
  return LaunchRowsByIndex<kTakeGradSorted>(dst, dstride, k_rows, sorted, index, index_is_int,
                                            n_index, src, sstride, cols, stream,
                                            "add_take_grad_large_batch");
}

int mshadow_hip_index_fill_f32(float *dst, int dstride, int k_rows, const void *index,
                               int index_is_int, int n_index, const float *src, int sstride,
                               int cols, void *stream) {
  const int chk = RowOpCheck(dst, dstride, k_rows, index, n_index, src, sstride, cols);
  if (chk != MSHADOW_HIP_OK) return chk < 0 ? MSHADOW_HIP_OK : chk;
  return LaunchRowsByIndex<kFill>(dst, dstride, k_rows, index, index, index_is_int, n_index, src,
                                  sstride, cols, stream, "index_fill");
}

/* ------------------------------------------------------------------ reductions */

int mshadow_hip_reduce_keep_lowest_f32(float *dst, const float *src, int sstride, int rows,
                                       int cols, int reducer, int saver, float scale,
                                       void *stream) {
  ABI_REQUIRE(rows >= 1, "can not reduce over empty tensor");
  ABI_REQUIRE(cols >= 0, "negative shape");
  if (cols == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL && src != NULL, "NULL tensor");
  ABI_REQUIRE(sstride >= cols, "pitch smaller than the row");
  RawPlan1D<float> d = {dst};
  RawPlan2D<const float> sp = {src, sstride};
  const unsigned grid = (cols + mshadow::hip::kLowestCols - 1) / mshadow::hip::kLowestCols;
  hipStream_t s = AsStream(stream);
  int st = DispatchReducer(reducer, [&](auto red) {
    return DispatchSaver(saver, [&](auto sv) {
      typedef decltype(red) R;
      typedef decltype(sv) S;
      if (rows >= kDmaMinRows) {
        hipLaunchKernelGGL((mshadow::hip::ReduceKeepLowestDmaKernel<S, R>), dim3(grid),
                           dim3(mshadow::hip::kDmaThreads), 0, s, dst, src,
                           static_cast<uint32_t>(sstride), static_cast<uint32_t>(rows),
                           static_cast<uint32_t>(cols), scale);
      } else if (rows >= 4096) {
        hipLaunchKernelGGL(
            (mshadow::hip::ReduceKeepLowestKernel<S, R, float, mshadow::hip::kRedBlockLarge,
                                                  RawPlan1D<float>, RawPlan2D<const float> >),
            dim3(grid), dim3(mshadow::hip::kRedBlockLarge), 0, s, d, sp,
            static_cast<uint32_t>(rows), static_cast<uint32_t>(cols), scale);
      } else {
        hipLaunchKernelGGL(
            (mshadow::hip::ReduceKeepLowestKernel<S, R, float, mshadow::hip::kRedBlockSmall,
                                                  RawPlan1D<float>, RawPlan2D<const float> >),
            dim3(grid), dim3(mshadow::hip::kRedBlockSmall), 0, s, d, sp,
            static_cast<uint32_t>(rows), static_cast<uint32_t>(cols), scale);
      }
      return MSHADOW_HIP_OK;
    });
  });
  if (st != MSHADOW_HIP_OK) return st;
  return AfterLaunch("reduce_keep_lowest");
}

int mshadow_hip_reduce_keep_highdim_f32(float *dst, const float *src, int sstride, int n, int c,
                                        int y, int x, int reducer, int saver, float scale,
                                        void *stream) {
  ABI_REQUIRE(n >= 0 && c >= 0 && y >= 0 && x >= 0, "negative shape");
  if (c == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL, "NULL tensor");
  ABI_REQUIRE(src != NULL || static_cast<long long>(n) * y * x == 0, "NULL tensor");
  ABI_REQUIRE(sstride >= x, "pitch smaller than the row");
  /* the kernels that stream a tensor from memory compute row numbers in 64 bits; the
     register-staged ones for short reductions (fewer than 2^16 values per kept index) in 32 */
  ABI_REQUIRE(static_cast<long long>(n) * c < (1ll << 31), "too many (n, c) segments for 32-bit indices");
  ABI_REQUIRE(static_cast<long long>(n) * c * y < (1ll << 31) ||
                  static_cast<long long>(n) * y * x >= kDmaMinPerKept,
              "too many rows for 32-bit indices");
  ABI_REQUIRE(static_cast<long long>(y) * x < (1ll << 31), "inner extent too large for 32-bit indices");
  RawPlan1D<float> d = {dst};
  RawPlan2D<const float> sp = {src, sstride};
  const mshadow::FastDivU32 div_x(static_cast<uint32_t>(x > 0 ? x : 1));
  hipStream_t s = AsStream(stream);
  /* The split kernel walks dense rows as one row per segment. It needs scratch memory for
     n * c inner results. */
  int v_y = y, v_x = x, v_stride = sstride;
  if (sstride == x) {
    v_x = v_stride = y * x;
    v_y = 1;
  }
  uint32_t *split_partial = NULL, *split_counter = NULL;
  /* With a kept index for (nearly) every CU the one-workgroup-per-kept-index kernel fills the
     chip and ends without a merge; with fewer the inner chains are dealt out by segments:
     16 per workgroup and a kilobyte of each per load where rows are whole 16-byte packs, else
     32 per workgroup and 256 bytes of each. */
  const bool few_kept = static_cast<long long>(c) * 4 < 3ll * mshadow_abi::ComputeUnits();
  const bool whole_packs = v_x % 4 == 0 && v_stride % 4 == 0 && Aligned16(src);
  if (few_kept && static_cast<long long>(n) * y * x >= kDmaMinPerKept &&
      static_cast<long long>(n) * c < (1ll << 31)) {
    const int sc = mshadow_hip_reduce_scratch(stream, static_cast<size_t>(n) * c, &split_partial,
                                              &split_counter);
    if (sc != MSHADOW_HIP_OK) return sc;
  }
  const mshadow::FastDivU32 v_div_x(static_cast<uint32_t>(v_x > 0 ? v_x : 1));
  int st = DispatchReducer(reducer, [&](auto red) {
    return DispatchSaver(saver, [&](auto sv) {
      typedef decltype(red) R;
      typedef decltype(sv) S;
#define HIGHDIM_LAUNCH_T(T, SEGS)                                                              \
  hipLaunchKernelGGL((mshadow::hip::ReduceKeepHighDimKernel<S, R, float, T, SEGS, RawPlan1D<float>, \
                                                            RawPlan2D<const float> >),         \
                     dim3(c), dim3(T), 0, s, d, sp, static_cast<uint32_t>(n),                  \
                     static_cast<uint32_t>(c), static_cast<uint32_t>(y),                       \
                     static_cast<uint32_t>(x), div_x, scale)
#define HIGHDIM_LAUNCH(SEGS)                                                                   \
  if (large)                                                                                   \
    hipLaunchKernelGGL((mshadow::hip::ReduceKeepHighDimDmaKernel<S, R, float, SEGS>), dim3(c),        \
                       dim3(mshadow::hip::kDmaThreads), 0, s, dst, src,                        \
                       static_cast<uint32_t>(sstride), static_cast<uint32_t>(n),               \
                       static_cast<uint32_t>(c), static_cast<uint32_t>(y),                     \
                       static_cast<uint32_t>(x), div_x, scale);                                \
  else HIGHDIM_LAUNCH_T(mshadow::hip::kRedBlockSmall, SEGS)
      const bool large = static_cast<long long>(n) * y * x >= kDmaMinPerKept;
      if (large && split_partial != NULL) {
#define HIGHDIM_SPLIT(RING)                                                                    \
  hipLaunchKernelGGL((mshadow::hip::ReduceKeepHighDimSplitKernel<S, R, float, RING>),          \
                     dim3((static_cast<unsigned>(n) * c + RING::kSegs - 1) / RING::kSegs),      \
                     dim3(RING::kThreads), 0, s, dst, src, static_cast<uint32_t>(v_stride),    \
                     static_cast<uint32_t>(n), static_cast<uint32_t>(c),                       \
                     static_cast<uint32_t>(v_y), static_cast<uint32_t>(v_x), v_div_x, scale,   \
                     split_partial, split_counter)
        if (whole_packs && static_cast<long long>(n) * c > 16ll * mshadow_abi::ComputeUnits()) {
          HIGHDIM_SPLIT(mshadow::hip::HighDimSplitRingPacksWide);
        } else if (whole_packs) {
          HIGHDIM_SPLIT(mshadow::hip::HighDimSplitRingPacks);
        } else {
          HIGHDIM_SPLIT(mshadow::hip::HighDimSplitRing);
        }
#undef HIGHDIM_SPLIT
        return MSHADOW_HIP_OK;
      }
      if (n > 16) { HIGHDIM_LAUNCH(64); }
      else if (n > 4) { HIGHDIM_LAUNCH(16); }
      else if (n > 1) { HIGHDIM_LAUNCH(4); }
      else { HIGHDIM_LAUNCH(1); }
#undef HIGHDIM_LAUNCH_T
#undef HIGHDIM_LAUNCH
      return MSHADOW_HIP_OK;
    });
  });
  if (st != MSHADOW_HIP_OK) return st;
  return AfterLaunch("reduce_keep_highdim");
}

/* ------------------------------------------------------------------ pool / unpool */

static const size_t kPoolLdsBudget = 48 * 1024;  // per workgroup: three resident per CU
static const size_t kUnpoolLdsBudget = 16 * 1024;  // smaller bands: more workgroups in different phases per CU

/*! \brief strips of the stride-1 unpool kernel over `rows` rows of `w` columns per plane:
 *  sixteen rows a strip, fewer while that leaves the machine short of waves */
static SlideGeom MakeSlideGeom(int planes, int rows, int w) {
  SlideGeom sg;
  sg.groups = static_cast<uint32_t>((w + 3) / 4);
  sg.strips_per_wave = 64u / sg.groups;
  uint32_t r = 16;
  const long long want = 16ll * mshadow_abi::ComputeUnits();  // waves
  while (r > 2 && static_cast<long long>(planes) * ((rows + r - 1) / r) / sg.strips_per_wave < want) r /= 2;
  sg.strip_rows = r;
  sg.strips_per_plane = static_cast<uint32_t>((rows + r - 1) / r);
  sg.total_strips = static_cast<uint32_t>(planes) * sg.strips_per_plane;
  sg.div_groups = mshadow::FastDivU32(sg.groups);
  sg.div_spp = mshadow::FastDivU32(sg.strips_per_plane);
  return sg;
}

int mshadow_hip_pool_f32(float *dst, int dstride, const float *src, int sstride, int planes,
                         int h, int w, int ph, int pw, int ky, int kx, int sy, int sx,
                         int reducer, void *stream) {
  ABI_REQUIRE(planes >= 0 && h >= 0 && w >= 0 && ph >= 0 && pw >= 0, "negative shape");
  ABI_REQUIRE(ky >= 1 && kx >= 1 && sy >= 1 && sx >= 1, "kernel and stride must be positive");
  ABI_REQUIRE(h >= ky && w >= kx, "kernel must be smaller than image");
  ABI_REQUIRE(reducer >= MSHADOW_HIP_SUM && reducer <= MSHADOW_HIP_MIN, "unknown reducer");
  if (planes == 0 || ph == 0 || pw == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL && src != NULL, "NULL tensor");
  ABI_REQUIRE(dstride >= pw && sstride >= w, "pitch smaller than the row");
  ABI_REQUIRE(static_cast<long long>(planes) * h < (1ll << 31) &&
                  static_cast<long long>(planes) * ph * pw < (1ll << 32),
              "too large for 32-bit indices");
  PoolGeom g = {h, w, ph, pw, ky, kx, sy, sx, 0, 0, w};
  hipStream_t s = AsStream(stream);
  const size_t row_bytes = static_cast<size_t>(g.lds_pitch) * sizeof(float);
  /* output rows per band so that (band - 1) * sy + ky input rows fit the budget */
  long long max_in_rows = static_cast<long long>(kPoolLdsBudget / row_bytes);
  long long band = max_in_rows >= ky ? (max_in_rows - ky) / sy + 1 : 0;
  if (band > ph) band = ph;
  /* keep at least ~4 workgroups per CU in flight when planes are few */
  while (band > 8 && static_cast<long long>(planes) * ((ph + band - 1) / band) < 1024) {
    band = (band + 1) / 2;
  }
  if (band >= 1) {
    /* equal-sized bands of about 20 KB of input rows (but four output rows or more): seven or
       eight workgroups then share a CU, and while some wait at their barrier others load.
       (32,64,224,224) 2x2 stride 2: 80 us against 102 us with bands of 41 KB; 14 KB and less
       lose again to the rows that neighbouring bands both read. */
    long long nb = (ph + band - 1) / band;
    const long long target = 20 * 1024;
    const long long want = (static_cast<long long>(ph) * sy * row_bytes + target - 1) / target;
    if (want > nb) nb = want;
    if (nb > ph / 4 && ph >= 4) nb = ph / 4;
    band = (ph + nb - 1) / nb;
  }
#define POOL_SWITCH(KERNEL, ...)                                                               \
  switch (reducer) {                                                                           \
    case MSHADOW_HIP_SUM: hipLaunchKernelGGL((KERNEL<MSHADOW_HIP_SUM>), __VA_ARGS__); break;    \
    case MSHADOW_HIP_MAX: hipLaunchKernelGGL((KERNEL<MSHADOW_HIP_MAX>), __VA_ARGS__); break;    \
    default: hipLaunchKernelGGL((KERNEL<MSHADOW_HIP_MIN>), __VA_ARGS__); break;                 \
  }
  /* small planes: several whole planes per workgroup, about 24 KB of them */
  const long long plane_bytes = static_cast<long long>(h) * row_bytes;
  if (plane_bytes * 2 <= 24 * 1024 && planes >= 2) {
    long long per_block = (24 * 1024) / plane_bytes;
    /* ... but no fewer workgroups than keep every CU busy four times over */
    while (per_block > 1 && (planes + per_block - 1) / per_block < 4ll * mshadow_abi::ComputeUnits()) {
      per_block = (per_block + 1) / 2;
    }
    if (per_block >= 2) {
      const size_t lds = static_cast<size_t>(per_block) * plane_bytes + 16;
      const unsigned blocks = static_cast<unsigned>((planes + per_block - 1) / per_block);
      const mshadow::FastDivU32 div_ph(static_cast<uint32_t>(ph));
#define POOL_PLANES(KY, KX)                                                                     \
  switch (reducer) {                                                                           \
    case MSHADOW_HIP_SUM:                                                                      \
      hipLaunchKernelGGL((PoolPlanesKernel<MSHADOW_HIP_SUM, KY, KX>), dim3(blocks), dim3(kPoolBlock), \
                         lds, s, dst, dstride, src, sstride, g, planes, static_cast<int>(per_block), div_ph); \
      break;                                                                                   \
    case MSHADOW_HIP_MAX:                                                                      \
      hipLaunchKernelGGL((PoolPlanesKernel<MSHADOW_HIP_MAX, KY, KX>), dim3(blocks), dim3(kPoolBlock), \
                         lds, s, dst, dstride, src, sstride, g, planes, static_cast<int>(per_block), div_ph); \
      break;                                                                                   \
    default:                                                                                   \
      hipLaunchKernelGGL((PoolPlanesKernel<MSHADOW_HIP_MIN, KY, KX>), dim3(blocks), dim3(kPoolBlock), \
                         lds, s, dst, dstride, src, sstride, g, planes, static_cast<int>(per_block), div_ph); \
      break;                                                                                   \
  }
      if (ky == 3 && kx == 3) { POOL_PLANES(3, 3) }
      else if (ky == 2 && kx == 2) { POOL_PLANES(2, 2) }
      else { POOL_PLANES(0, 0) }
#undef POOL_PLANES
      return AfterLaunch("pool");
    }
  }
  if (band >= 1) {
    g.band = static_cast<int>(band);
    g.bands = (ph + g.band - 1) / g.band;
    const size_t lds = (static_cast<size_t>(g.band - 1) * sy + ky) * row_bytes + 16;
    const long long blocks = static_cast<long long>(planes) * g.bands;
    ABI_REQUIRE(blocks < (1ll << 31), "too many workgroups");
    /* windows that move by one element: a thread walks down an output column, KX reads of LDS an
       output. The band's rows are cut into `nruns` runs so that the columns of all runs fill the
       workgroup's threads in as few, as short rounds as can be. */
    if (sy == 1 && sx == 1 && ky == kx && (ky == 2 || ky == 3 || ky == 5) && ph <= h - ky + 1 &&
        pw <= w - kx + 1) {
      int nruns = 1, run_len = g.band;
      long long best = -1;
      for (int n = 1; n <= g.band; ++n) {
        const int rl = (g.band + n - 1) / n;
        const long long rounds = (static_cast<long long>(n) * pw + kPoolBlock - 1) / kPoolBlock;
        const long long cost = rounds * (rl + ky - 1);
        if (best < 0 || cost < best) { best = cost; nruns = n; run_len = rl; }
      }
      const mshadow::FastDivU32 div_pw(static_cast<uint32_t>(pw));
#define POOL_COLUMNS(K)                                                                        \
  switch (reducer) {                                                                           \
    case MSHADOW_HIP_SUM:                                                                      \
      hipLaunchKernelGGL((PoolColumnsS1Kernel<MSHADOW_HIP_SUM, K, K>), dim3(static_cast<unsigned>(blocks)), \
                         dim3(kPoolBlock), lds, s, dst, dstride, src, sstride, g, nruns, run_len, div_pw); \
      break;                                                                                   \
    case MSHADOW_HIP_MAX:                                                                      \
      hipLaunchKernelGGL((PoolColumnsS1Kernel<MSHADOW_HIP_MAX, K, K>), dim3(static_cast<unsigned>(blocks)), \
                         dim3(kPoolBlock), lds, s, dst, dstride, src, sstride, g, nruns, run_len, div_pw); \
      break;                                                                                   \
    default:                                                                                   \
      hipLaunchKernelGGL((PoolColumnsS1Kernel<MSHADOW_HIP_MIN, K, K>), dim3(static_cast<unsigned>(blocks)), \
                         dim3(kPoolBlock), lds, s, dst, dstride, src, sstride, g, nruns, run_len, div_pw); \
      break;                                                                                   \
  }
      if (ky == 2) { POOL_COLUMNS(2) }
      else if (ky == 3) { POOL_COLUMNS(3) }
      else { POOL_COLUMNS(5) }
#undef POOL_COLUMNS
      return AfterLaunch("pool");
    }
#define POOL_TILED(KY, KX)                                                                     \
  switch (reducer) {                                                                           \
    case MSHADOW_HIP_SUM:                                                                      \
      hipLaunchKernelGGL((PoolKernel<MSHADOW_HIP_SUM, KY, KX>), dim3(static_cast<unsigned>(blocks)), \
                         dim3(kPoolBlock), lds, s, dst, dstride, src, sstride, g);             \
      break;                                                                                   \
    case MSHADOW_HIP_MAX:                                                                      \
      hipLaunchKernelGGL((PoolKernel<MSHADOW_HIP_MAX, KY, KX>), dim3(static_cast<unsigned>(blocks)), \
                         dim3(kPoolBlock), lds, s, dst, dstride, src, sstride, g);             \
      break;                                                                                   \
    default:                                                                                   \
      hipLaunchKernelGGL((PoolKernel<MSHADOW_HIP_MIN, KY, KX>), dim3(static_cast<unsigned>(blocks)), \
                         dim3(kPoolBlock), lds, s, dst, dstride, src, sstride, g);             \
      break;                                                                                   \
  }
    if (ky == 3 && kx == 3) { POOL_TILED(3, 3) }
    else if (ky == 2 && kx == 2) { POOL_TILED(2, 2) }
    else { POOL_TILED(0, 0) }
#undef POOL_TILED
  } else {
    const unsigned total = static_cast<unsigned>(planes) * ph * pw;
    unsigned grid = 0;
    int st = mshadow_hip_suggest_grid(total, kPoolBlock, 4, &grid);
    if (st != MSHADOW_HIP_OK) return st;
    POOL_SWITCH(PoolDirectKernel, dim3(grid), dim3(kPoolBlock), 0, s, dst, dstride, src, sstride,
                g, total)
  }
  return AfterLaunch("pool");
}

int mshadow_hip_unpool_f32(float *dst, int dstride, const float *src, int sstride,
                           const float *pooled, int pstride, const float *grad, int gstride,
                           int planes, int h, int w, int ph, int pw, int ky, int kx, int sy,
                           int sx, int reducer, void *stream) {
  ABI_REQUIRE(planes >= 0 && h >= 0 && w >= 0 && ph >= 0 && pw >= 0, "negative shape");
  ABI_REQUIRE(ky >= 1 && kx >= 1 && sy >= 1 && sx >= 1, "kernel and stride must be positive");
  ABI_REQUIRE(reducer >= MSHADOW_HIP_SUM && reducer <= MSHADOW_HIP_MIN, "unknown reducer");
  if (planes == 0 || h == 0 || w == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL && src != NULL, "NULL tensor");
  ABI_REQUIRE((pooled != NULL && grad != NULL) || ph == 0 || pw == 0, "NULL tensor");
  ABI_REQUIRE(dstride >= w && sstride >= w && pstride >= pw && gstride >= pw,
              "pitch smaller than the row");
  ABI_REQUIRE(static_cast<long long>(planes) * h * w < (1ll << 32) &&
                  static_cast<long long>(planes) * h < (1ll << 31),
              "too large for 32-bit indices");
  PoolGeom g = {h, w, ph, pw, ky, kx, sy, sx, 0, 0, pw};
  hipStream_t s = AsStream(stream);
  /* 3 x 3 windows with stride 2 on rows of up to 256 pixels: no staging. Even heights and rows of
     whole aligned packs take the plain form, everything else the one that moves packs anywhere */
  if (ky == 3 && kx == 3 && sy == 2 && sx == 2 && w <= 256 && ph >= 1 && pw >= 1 &&
      static_cast<long long>(planes) * ph * pw >= 2) {
    const bool whole = h % 2 == 0 && w % 4 == 0 && dstride % 4 == 0 && sstride % 4 == 0 &&
                       Aligned16(dst) && Aligned16(src);
    UnpoolRowsGeom rg;
    rg.half_h = static_cast<uint32_t>((h + 1) / 2);
    rg.total_rows = static_cast<uint32_t>(planes) * rg.half_h;
    rg.groups = static_cast<uint32_t>((w + 3) / 4);
    rg.rows_per_wave = 64u / rg.groups;
    rg.div_groups = mshadow::FastDivU32(rg.groups);
    rg.div_half_h = mshadow::FastDivU32(rg.half_h);
    rg.pooled_floats = (static_cast<size_t>(planes) * ph - 1) * pstride + pw;
    rg.grad_floats = (static_cast<size_t>(planes) * ph - 1) * gstride + pw;
    rg.src_floats = (static_cast<size_t>(planes) * h - 1) * sstride + w;
    const uint32_t waves = (rg.total_rows + rg.rows_per_wave - 1) / rg.rows_per_wave;
    const uint32_t blocks = (waves + kPoolBlock / 64 - 1) / (kPoolBlock / 64);
#define UNPOOL_ROWS(R)                                                                          \
  do {                                                                                          \
    if (whole) {                                                                                \
      hipLaunchKernelGGL((UnpoolRows3x3s2Kernel<R, false>), dim3(blocks), dim3(kPoolBlock), 0, s, dst, \
                         dstride, src, sstride, pooled, pstride, grad, gstride, g, rg);         \
    } else {                                                                                    \
      hipLaunchKernelGGL((UnpoolRows3x3s2Kernel<R, true>), dim3(blocks), dim3(kPoolBlock), 0, s, dst, \
                         dstride, src, sstride, pooled, pstride, grad, gstride, g, rg);         \
    }                                                                                           \
  } while (0)
    if (reducer == MSHADOW_HIP_SUM) UNPOOL_ROWS(MSHADOW_HIP_SUM);
    else if (reducer == MSHADOW_HIP_MAX) UNPOOL_ROWS(MSHADOW_HIP_MAX);
    else UNPOOL_ROWS(MSHADOW_HIP_MIN);
#undef UNPOOL_ROWS
    return AfterLaunch("unpool");
  }
  /* 2 x 2 and 3 x 3 windows with stride 1 on planes of 64 to 256 pixels a side: no staging, the
     pooled rows over the current source row in registers ((128,64,112,112): 368 us against 513 us
     for the kernels below; on planes of 57 x 57 the two are level, below that the staged ones win) */
  if (ky == kx && (ky == 2 || ky == 3 || ky == 5) && sy == 1 && sx == 1 && w >= 64 && w <= 256 && h >= 64 && ph >= 1 && pw >= 1 &&
      static_cast<long long>(planes) * ph * pw >= 4 && static_cast<long long>(planes) * ((h + 1) / 2) < (1ll << 31)) {
    SlideGeom sg = MakeSlideGeom(planes, h, w);
    sg.src_floats = (static_cast<size_t>(planes) * h - 1) * sstride + w;
    sg.pooled_floats = (static_cast<size_t>(planes) * ph - 1) * pstride + pw;
    sg.grad_floats = (static_cast<size_t>(planes) * ph - 1) * gstride + pw;
    const uint32_t waves = (sg.total_strips + sg.strips_per_wave - 1) / sg.strips_per_wave;
    const uint32_t blocks = (waves + kPoolBlock / 64 - 1) / (kPoolBlock / 64);
#define UNPOOL_SLIDE(R)                                                                        \
  do {                                                                                         \
    if (ky == 2) {                                                                             \
      hipLaunchKernelGGL((UnpoolSlideS1Kernel<R, 2, 4>), dim3(blocks), dim3(kPoolBlock), 0, s, dst, dstride, \
                         src, sstride, pooled, pstride, grad, gstride, g, sg);                 \
    } else if (ky == 3) {                                                                      \
      hipLaunchKernelGGL((UnpoolSlideS1Kernel<R, 3, 3>), dim3(blocks), dim3(kPoolBlock), 0, s, dst, dstride, \
                         src, sstride, pooled, pstride, grad, gstride, g, sg);                 \
    } else {                                                                                   \
      hipLaunchKernelGGL((UnpoolSlideS1Kernel<R, 5, 5>), dim3(blocks), dim3(kPoolBlock), 0, s, dst, dstride, \
                         src, sstride, pooled, pstride, grad, gstride, g, sg);                 \
    }                                                                                          \
  } while (0)
    if (reducer == MSHADOW_HIP_SUM) UNPOOL_SLIDE(MSHADOW_HIP_SUM);
    else if (reducer == MSHADOW_HIP_MAX) UNPOOL_SLIDE(MSHADOW_HIP_MAX);
    else UNPOOL_SLIDE(MSHADOW_HIP_MIN);
#undef UNPOOL_SLIDE
    return AfterLaunch("unpool");
  }
  /* 2 x 2 windows, stride 2: a pixel has one window at most; four pixels and two windows per thread */
  if (ky == 2 && kx == 2 && sy == 2 && sx == 2 && w >= 4) {
    const long long wpk = (w + 3) / 4;
    const long long packs = static_cast<long long>(planes) * h * wpk;
    if (packs + kPoolBlock < (1ll << 31)) {
      const unsigned blocks = static_cast<unsigned>((packs + kPoolBlock - 1) / kPoolBlock);
      POOL_SWITCH(Unpool2x2s2Kernel, dim3(blocks), dim3(kPoolBlock), 0, s, dst, dstride, src, sstride,
                  pooled, pstride, grad, gstride, g, mshadow::FastDivU32(static_cast<uint32_t>(wpk)),
                  mshadow::FastDivU32(static_cast<uint32_t>(h)), static_cast<uint32_t>(packs))
      return AfterLaunch("unpool");
    }
  }
  /* small planes under a stride of 2 or more (a pixel has few windows): no staging. Measured on
     (128,256,28,28), 2x2 stride 2: 56 us against 96 us for the kernels below; on large planes or
     with stride 1 the staged kernels are faster. */
  if (static_cast<long long>(h) * w * sizeof(float) <= 4 * 1024 && sy >= 2 && sx >= 2 && w >= 4) {
    const long long wpk = (w + 3) / 4;
    const long long packs = static_cast<long long>(planes) * h * wpk;
    if (packs + kPoolBlock < (1ll << 31)) {
      const unsigned blocks = static_cast<unsigned>((packs + kPoolBlock - 1) / kPoolBlock);
      POOL_SWITCH(UnpoolGatherKernel, dim3(blocks), dim3(kPoolBlock), 0, s, dst, dstride, src, sstride,
                  pooled, pstride, grad, gstride, g, mshadow::FastDivU32(static_cast<uint32_t>(sy)),
                  mshadow::FastDivU32(static_cast<uint32_t>(sx)),
                  mshadow::FastDivU32(static_cast<uint32_t>(wpk)),
                  mshadow::FastDivU32(static_cast<uint32_t>(h)), static_cast<uint32_t>(packs))
      return AfterLaunch("unpool");
    }
  }
  /* small planes: several whole planes per workgroup (about 24 KB of pooled values and gradients) */
  {
    const long long plane_bytes = static_cast<long long>(ph) * g.lds_pitch * sizeof(float) * 2;
    const long long src_plane_bytes = static_cast<long long>(h) * w * sizeof(float);
    if (plane_bytes > 0 && plane_bytes * 2 <= 24 * 1024 && src_plane_bytes <= 4 * 1024 && planes >= 2) {
      long long per_block = (24 * 1024) / plane_bytes;
      while (per_block > 1 &&
             (planes + per_block - 1) / per_block < 4ll * mshadow_abi::ComputeUnits()) {
        per_block = (per_block + 1) / 2;
      }
      if (per_block >= 2) {
        const size_t lds = static_cast<size_t>(per_block) * plane_bytes + 32;
        const unsigned blocks = static_cast<unsigned>((planes + per_block - 1) / per_block);
        const mshadow::FastDivU32 div_h(static_cast<uint32_t>(h));
#define UNPOOL_PLANES(KY, KX, SY, SX)                                                          \
  switch (reducer) {                                                                           \
    case MSHADOW_HIP_SUM:                                                                      \
      hipLaunchKernelGGL((UnpoolPlanesKernel<MSHADOW_HIP_SUM, KY, KX, SY, SX>), dim3(blocks),   \
                         dim3(kPoolBlock), lds, s, dst, dstride, src, sstride, pooled, pstride, \
                         grad, gstride, g, planes, static_cast<int>(per_block), div_h);        \
      break;                                                                                   \
    case MSHADOW_HIP_MAX:                                                                      \
      hipLaunchKernelGGL((UnpoolPlanesKernel<MSHADOW_HIP_MAX, KY, KX, SY, SX>), dim3(blocks),   \
                         dim3(kPoolBlock), lds, s, dst, dstride, src, sstride, pooled, pstride, \
                         grad, gstride, g, planes, static_cast<int>(per_block), div_h);        \
      break;                                                                                   \
    default:                                                                                   \
      hipLaunchKernelGGL((UnpoolPlanesKernel<MSHADOW_HIP_MIN, KY, KX, SY, SX>), dim3(blocks),   \
                         dim3(kPoolBlock), lds, s, dst, dstride, src, sstride, pooled, pstride, \
                         grad, gstride, g, planes, static_cast<int>(per_block), div_h);        \
      break;                                                                                   \
  }
        if (ky == 3 && kx == 3 && sy == 2 && sx == 2) { UNPOOL_PLANES(3, 3, 2, 2) }
        else if (ky == 2 && kx == 2 && sy == 2 && sx == 2) { UNPOOL_PLANES(2, 2, 2, 2) }
        else if (ky == 3 && kx == 3 && sy == 1 && sx == 1) { UNPOOL_PLANES(3, 3, 1, 1) }
        else { UNPOOL_PLANES(0, 0, 0, 0) }
#undef UNPOOL_PLANES
        return AfterLaunch("unpool");
      }
    }
  }
  const size_t row_bytes = static_cast<size_t>(g.lds_pitch) * sizeof(float) * 2;  // pooled + grad
  /* source rows per band: prow_max = (band + ky - 2) / sy + 2 pooled rows must fit */
  long long max_prow = static_cast<long long>(kUnpoolLdsBudget / row_bytes);
  long long band = (max_prow - 2) * sy - ky + 2;
  if (band > h) band = h;
  while (band > 8 && static_cast<long long>(planes) * ((h + band - 1) / band) < 1024) {
    band = (band + 1) / 2;
  }
  if (band >= 1) {  // equal-sized bands, starting at multiples of the stride
    const long long nb = (h + band - 1) / band;
    band = (h + nb - 1) / nb;
    band = (band + sy - 1) / sy * sy;
  }
  if (band >= 1 && max_prow >= 3) {
    g.band = static_cast<int>(band);
    g.bands = (h + g.band - 1) / g.band;
    const int prow_max = (g.band + ky - 2) / sy + 2;
    const size_t lds = static_cast<size_t>(prow_max) * row_bytes + 32;
    const long long blocks = static_cast<long long>(planes) * g.bands;
    ABI_REQUIRE(blocks < (1ll << 31), "too many workgroups");
    ABI_REQUIRE(lds <= 160 * 1024, "pooled rows too long for the LDS-tiled kernel");
    const mshadow::FastDivU32 div_bw(static_cast<uint32_t>((w + sx - 1) / sx));
    /* whole, aligned blocks of sx pixels per row: a block row is one memory access */
    const bool vec = (sx == 2 || sx == 4) && w % sx == 0 && dstride % sx == 0 && sstride % sx == 0 &&
                     reinterpret_cast<uintptr_t>(dst) % (sx * 4) == 0 &&
                     reinterpret_cast<uintptr_t>(src) % (sx * 4) == 0;
    const UnpoolArgs ua = {dst, dstride, src, sstride, pooled, pstride, grad, gstride, g, prow_max,
                           static_cast<unsigned>(blocks), lds, s};
    if (ky == 3 && kx == 3 && sy == 2 && sx == 2) {
      if (vec) LaunchUnpoolBlock<3, 3, 2, 2, true>(reducer, ua, div_bw);
      else LaunchUnpoolBlock<3, 3, 2, 2, false>(reducer, ua, div_bw);
    } else if (ky == 2 && kx == 2 && sy == 2 && sx == 2) {
      if (vec) LaunchUnpoolBlock<2, 2, 2, 2, true>(reducer, ua, div_bw);
      else LaunchUnpoolBlock<2, 2, 2, 2, false>(reducer, ua, div_bw);
    } else if (ky == 3 && kx == 3 && sy == 1 && sx == 1) {
      LaunchUnpoolBlock<3, 3, 1, 1, false>(reducer, ua, div_bw);
    } else {
      LaunchUnpoolGeneric(reducer, ua);
    }
  } else {
    const unsigned total = static_cast<unsigned>(planes) * h * w;
    unsigned grid = 0;
    int st = mshadow_hip_suggest_grid(total, kPoolBlock, 4, &grid);
    if (st != MSHADOW_HIP_OK) return st;
    POOL_SWITCH(UnpoolDirectKernel, dim3(grid), dim3(kPoolBlock), 0, s, dst, dstride, src,
                sstride, pooled, pstride, grad, gstride, g, total)
  }
#undef POOL_SWITCH
  return AfterLaunch("unpool");
}

/* ------------------------------------------------------------------ im2col / col2im */

#define PATCH_ENTRY(NAME, T, FN, A, AS, B, BS)                                                 \
  int NAME(T *A, int AS, const T *B, int BS, int n, int c, int h, int w, int ky, int kx, int sy, \
           int sx, int dy, int dx, int pad_y, int pad_x, void *stream) {                        \
    PatchGeom g;                                                                               \
    int st = MakePatchGeom(&g, n, c, h, w, ky, kx, sy, sx, dy, dx, pad_y, pad_x);              \
    if (st != MSHADOW_HIP_OK) return st;                                                       \
    return FN<T>(A, AS, B, BS, g, stream);                                                     \
  }
PATCH_ENTRY(mshadow_hip_im2col_f16, uint16_t, Im2Col, col, cstride, img, istride)
PATCH_ENTRY(mshadow_hip_im2col_f32, float, Im2Col, col, cstride, img, istride)
PATCH_ENTRY(mshadow_hip_col2im_f16, uint16_t, Col2Im, img, istride, col, cstride)
PATCH_ENTRY(mshadow_hip_col2im_f32, float, Col2Im, img, istride, col, cstride)
#undef PATCH_ENTRY

}  // extern "C"
