/*
 * Elementwise evaluation kernels: Saver::Save(dst(y, x), plan.Eval(y, x)) for every
 * element of the destination's 2-D view. They replace MapPlanKernel /
 * MapPlanLargeKernel of the reference (mshadow/cuda/tensor_gpu-inl.cuh:67-120), which
 * handle one element per thread with a division per element and 4-byte accesses.
 *
 * MapPackKernel  every leaf evaluates packs: each thread moves kPackUnroll packs of N = 16 /
 *                sizeof(DType) elements with one 128-bit global access per leaf, wherever the
 *                pack lies (no alignment is needed). Plans of tensors, scalars and elementwise
 *                functions also take rows that are not whole packs (the last pack of a row
 *                element by element); other packable plans need cols % N == 0. When
 *                all rows are dense the 2-D view is walked linearly and no division
 *                is executed at all; otherwise there is one per pack. Large tensors are
 *                moved with non-temporal accesses (measured on MI355X: 6.3 TB/s against
 *                5.6 TB/s with default cache policy for a 4-in 1-out map).
 *                Algorithmic traffic: (leaves + 1) * sizeof(DType) bytes per element,
 *                HBM-bound (5 * 4 B for dst = A*B + 0.5f*F<sigmoid>(C) - D).
 * MapScalarKernel any plan (chainers, transposes, caller-defined plans, unaligned or
 *                ragged rows): one element per thread-iteration, grid-stride; the split of
 *                the flat index into (row, column) is a multiply-high.
 */
#ifndef MSHADOW_HIP_KERNELS_MAP_H_
#define MSHADOW_HIP_KERNELS_MAP_H_

#include "../../core/fastdiv.h"
#include "../../expr/plan.h"
#include "./common.h"

namespace mshadow {
namespace hip {

const int kMapBlock = 256;
/*! \brief packs per thread; the loads of all of them are issued before the first use.
 *  One pack per thread and many small workgroups serve a one- or two-tensor map best
 *  (MI355X: dst = src over 8192x32000 floats 337 us against 353 us with four packs;
 *  dst = x + broadcast<1>(bias) over (64,256,56,56) 70 us against 80 us); an expression
 *  that reads three tensors or more takes four (the 4-in 1-out map: 57 us, 58-59 us
 *  with two or eight). */
const int kPackUnroll = 1;
const int kPackUnrollDeep = 4;

/*! \brief PER consecutive elements of one row per thread-iteration (PER divides cols): the
 *  PER evaluations are independent, so their loads are in flight together, and where a
 *  plan reads consecutive addresses the compiler merges them into one wide load. */
template <typename Saver, typename DType, typename DPlan, typename SPlan, int PER>
__global__ void __launch_bounds__(kMapBlock)
    MapScalarKernel(DPlan dplan, SPlan splan, uint32_t rows, uint32_t cols, FastDivU32 div_cols,
                    uint32_t row0) {
  /* one launch covers `rows` rows from row0 on, fewer than 2^31 elements; a larger view is
     covered by several launches */
  const uint32_t total = rows * cols;
  const uint32_t step = gridDim.x * kMapBlock * PER;
  const uint32_t piece = StripOfBlock(blockIdx.x, gridDim.x);
  for (uint32_t i = (piece * kMapBlock + threadIdx.x) * PER; i < total; i += step) {
    const uint32_t yr = div_cols.Div(i);  // a multiply-high, not a hardware division
    const uint32_t x = i - yr * cols;
    const uint32_t y = yr + row0;
    DType v[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) v[k] = splan.Eval(y, x + k);
#pragma unroll
    for (int k = 0; k < PER; ++k) Saver::template Save<DType>(dplan.REval(y, x + k), v[k]);
  }
}

/*! \brief the store half of the pack kernels */
template <typename Saver, typename DType, int N, bool kStream, typename DPlan>
__device__ __forceinline__ void SavePack(DPlan &dplan, uint32_t y, uint32_t x,
                                         const expr::Pack<DType, N> &val) {
  typedef expr::Pack<DType, N> P;
  if (SaverReadsDst<Saver>::value) {
    P old = dplan.template EvalPack<N, kStream>(y, x);
#pragma unroll
    for (int i = 0; i < N; ++i) Saver::template Save<DType>(old.v[i], val.v[i]);
    dplan.template StorePack<N, kStream>(y, x, old);
  } else {
    dplan.template StorePack<N, kStream>(y, x, val);
  }
}

/*! \brief row_elems: elements of a row (of the whole run when kFlat). Where it is not a multiple
 *  of N the last pack of a row (of the run) is partial and is evaluated element by element;
 *  only plans of tensors, scalars and elementwise functions are launched that way. */
template <typename Saver, typename DType, int N, bool kFlat, bool kStream, int kPackUnroll,
          typename DPlan, typename SPlan>
__global__ void __launch_bounds__(kMapBlock)
    MapPackKernel(DPlan dplan, SPlan splan, uint32_t total_packs, uint32_t packs_per_row,
                  FastDivU32 div_ppr, uint32_t row0, uint32_t row_elems) {
  typedef expr::Pack<DType, N> P;
  /* with real row numbers in play (windows over rows re-read their neighbours' data), each
     XCD takes a contiguous run of the workgroups */
  const uint32_t block = kFlat ? blockIdx.x : StripOfBlock(blockIdx.x, gridDim.x);
  const uint32_t base = block * (kMapBlock * kPackUnroll) + threadIdx.x;
  uint32_t y[kPackUnroll], x[kPackUnroll];
  P val[kPackUnroll];
#pragma unroll
  for (int u = 0; u < kPackUnroll; ++u) {
    const uint32_t p = base + u * kMapBlock;
    if (kFlat) {
      y[u] = 0;
      x[u] = p * N;
    } else {
      const uint32_t yr = div_ppr.Div(p);
      x[u] = (p - yr * packs_per_row) * N;
      y[u] = yr + row0;  // the launch covers whole rows from row0 on, fewer than 2^31 packs
    }
    if (p < total_packs) {
      if (x[u] + N <= row_elems) {
        val[u] = splan.template EvalPack<N, kStream>(y[u], x[u]);
      } else {
#pragma unroll
        for (int i = 0; i < N; ++i) {
          if (x[u] + i < row_elems) val[u].v[i] = splan.Eval(y[u], x[u] + i);
        }
      }
    }
  }
#pragma unroll
  for (int u = 0; u < kPackUnroll; ++u) {
    const uint32_t p = base + u * kMapBlock;
    if (p < total_packs) {
      if (x[u] + N <= row_elems) {
        SavePack<Saver, DType, N, kStream>(dplan, y[u], x[u], val[u]);
      } else {
#pragma unroll
        for (int i = 0; i < N; ++i) {
          if (x[u] + i < row_elems) Saver::template Save<DType>(dplan.REval(y[u], x[u] + i), val[u].v[i]);
        }
      }
    }
  }
}

/*! \brief the pack kernel for plans with a window over neighbouring planes (channel
 *  pooling): a plane is plane_rows rows of packs_per_row packs, a workgroup is a run of
 *  kMapBlock packs through kPackUnroll adjacent planes, and a thread evaluates the same
 *  place of those planes in one call, so that overlapping windows share their fetches.
 *  Workgroups of one group of planes are neighbours in the grid: what two groups both read
 *  is still in L2 (measured for x * (chpool<sum>(x * x, 5) * a + 1) over (64,256,56,56):
 *  226 MiB fetched against 463 MiB in linear order, 196 MiB needed). */
template <typename Saver, typename DType, int N, bool kStream, int kPackUnroll, typename DPlan,
          typename SPlan>
__global__ void __launch_bounds__(kMapBlock)
    MapPackPlanesKernel(DPlan dplan, SPlan splan, uint32_t total_packs, uint32_t packs_per_row,
                        FastDivU32 div_ppr, uint32_t plane_rows, FastDivU32 div_plane_packs) {
  typedef expr::Pack<DType, N> P;
  const uint32_t plane_packs = div_plane_packs.div;
  const uint32_t block = StripOfBlock(blockIdx.x, gridDim.x);
  /* threads count the places of all groups of planes in one sequence */
  const uint32_t place = block * kMapBlock + threadIdx.x;
  const uint32_t group = div_plane_packs.Div(place);
  const uint32_t at = place - group * plane_packs;
  const uint32_t first = group * kPackUnroll * plane_packs + at;  // pack in the first plane
  if (first >= total_packs) return;
  const uint32_t y0 = div_ppr.Div(first);
  const uint32_t x = (first - y0 * packs_per_row) * N;
  P val[kPackUnroll];
  if (first + (kPackUnroll - 1) * plane_packs < total_packs) {
    /* what one plan node fetches another may fetch again (the centre of a window is often a
       leaf of its own): ordinary loads throughout, streaming only for the stores */
    expr::EvalPackRun<N, false, kPackUnroll>(splan, y0, plane_rows, x, val);
#pragma unroll
    for (int u = 0; u < kPackUnroll; ++u) {
      SavePack<Saver, DType, N, kStream>(dplan, y0 + u * plane_rows, x, val[u]);
    }
  } else {  // the last group of planes is short
    for (int u = 0; u < kPackUnroll && first + u * plane_packs < total_packs; ++u) {
      const P one = splan.template EvalPack<N, false>(y0 + u * plane_rows, x);
      SavePack<Saver, DType, N, kStream>(dplan, y0 + u * plane_rows, x, one);
    }
  }
}

}  // namespace hip
}  // namespace mshadow
#endif  // MSHADOW_HIP_KERNELS_MAP_H_
