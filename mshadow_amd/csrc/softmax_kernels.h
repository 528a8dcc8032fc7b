/*
 * Row softmax and its gradient for gfx950.
 *
 * SoftmaxRowKernel: one workgroup per row, the whole row held in registers, so HBM
 * sees one read of src and one write of dst (2 * 4 bytes per element; the reference
 * kernel, mshadow/cuda/tensor_gpu-inl.cuh:330-393, moves 5). Steps per row:
 *   1. 128-bit loads, row maximum by DPP wave reduction + one LDS exchange;
 *   2. p = exp(x - max) in registers (hardware exp2 with a compensated argument);
 *   3. the row sum in the CPU path's left-to-right order (ordered_sum.h), so that the
 *      sum is, bit for bit, what mshadow/tensor_cpu-inl.h:277-281 computes from the same p;
 *   4. p / sum (reciprocal and one correction step), 128-bit stores.
 * dst may alias src (every element is read before the row is written).
 * SoftmaxLongRowKernel covers rows too long for registers with the same arithmetic,
 * staging p through dst. SoftmaxGradKernel is a 128-bit copy with one element per row
 * decremented (mshadow/tensor_cpu-inl.h:287-302).
 */
#ifndef MSHADOW_AMD_CSRC_SOFTMAX_KERNELS_H_
#define MSHADOW_AMD_CSRC_SOFTMAX_KERNELS_H_

#include <hip/hip_runtime.h>

#include <mshadow/hip/kernels/common.h>

#include "ordered_sum.h"
#include "stream_access.h"

namespace mshadow_hipk {

using mshadow::hip::kWave;
using mshadow::hip::LaneId;
using mshadow::hip::ReadLaneF32;
using mshadow::hip::WaveId;
using mshadow::hip::WaveInclusiveScanF32;
using mshadow::hip::WaveMaxF32;

/*! \brief LDS scratch of the ordered sum: two alternating sets of per-wave totals and
 *  the hand-over slot for the running sum */
template <int WAVES>
struct OrderedSumLds {
  float q[2][WAVES];
  float s;
  float wmax[WAVES];
};

/*! \brief one wave adds its 64 * N terms (lane order, then element order) to s exactly
 *  as a serial loop would; called only for the wave in which a chunk was rejected */
template <int N>
__device__ inline float WaveResolve(float s, const float (&t)[N]) {
  using namespace ordered_sum;
  const int lane = LaneId();
  int start = 0;
  while (true) {
    const Binade b = BinadeOf(s);
    const float q = (lane >= start) ? LaneQuant<N>(t, b) : 0.0f;
    const float incl = WaveInclusiveScanF32(q);
    const bool fail = (lane >= start) && !Fits(b, incl);
    const unsigned long long mask = __ballot(fail);
    if (mask == 0ull) return Accept(s, b, ReadLaneF32(incl, kWave - 1));
    const int first = __ffsll(mask) - 1;
    /* lanes before `first` are exact integer adds (their inclusive prefix is exact) */
    s = Accept(s, b, first > 0 ? ReadLaneF32(incl, first - 1) : 0.0f);
    /* lane `first` does real float adds; every lane computes, one result is taken */
    s = ReadLaneF32(TrueAdd<N>(s, t), first);
    start = first + 1;
    if (start == kWave) return s;
  }
}

/*! \brief block-wide: add one slab (THREADS * N consecutive terms, thread-major) to s.
 *  s is uniform over the block on entry and on exit. `buf` alternates the LDS slot. */
template <int THREADS, int N>
__device__ inline float BlockOrderedAdd(float s, const float (&t)[N],
                                        OrderedSumLds<THREADS / kWave> *lds, int *buf) {
  using namespace ordered_sum;
  const int W = THREADS / kWave;
  const int wave = WaveId();
  const int lane = LaneId();
  int pos = 0;  // waves before pos are already in s
  while (true) {
    const Binade b = BinadeOf(s);
    if (wave >= pos) {
      const float q = ReadLaneF32(WaveInclusiveScanF32(LaneQuant<N>(t, b)), kWave - 1);
      if (lane == 0) lds->q[*buf][wave] = q;
    }
    __syncthreads();
    /* the per-wave totals are scanned across lanes (lane w holds wave w's total): the
       first wave whose inclusive prefix leaves the binade is the one to resolve */
    const float qv = (lane < W && lane >= pos) ? lds->q[*buf][lane] : 0.0f;
    const float incl = WaveInclusiveScanF32(qv);
    const bool over = lane < W && lane >= pos && !Fits(b, incl);
    const unsigned long long mask = __ballot(over);
    const int failw = mask ? __ffsll(mask) - 1 : W;
    const float acc = failw > 0 ? ReadLaneF32(incl, failw - 1) : 0.0f;
    *buf ^= 1;
    s = Accept(s, b, acc);
    if (failw == W) return s;
    if (wave == failw) {
      const float r = WaveResolve<N>(s, t);
      if (lane == 0) lds->s = r;
    }
    __syncthreads();
    s = lds->s;
    pos = failw + 1;
    if (pos == W) return s;
  }
}

/*! \brief e^x for x <= 0 (any float accepted): 2^(x * log2 e) with the rounding error of
 *  the product carried separately, so the result stays within about 1.5 ulp for the whole
 *  range a softmax sees. The hardware exp2 does not return subnormals, so results below
 *  2^-126 are computed 64 binades up and scaled back. */
__device__ __forceinline__ float ExpNonPositive(float x) {
  const float kLog2eHi = 1.44269502162933349609375f;
  const float kLog2eLo = 1.925963033500011079013347625732421875e-08f;
  const float t = x * kLog2eHi;
  float r = __builtin_fmaf(x, kLog2eHi, -t);   // exact rounding error of the product
  r = __builtin_fmaf(x, kLog2eLo, r);
  if (__builtin_expect(!(t >= -125.0f), 0)) {   // subnormal / zero result, -inf, NaN
    if (t < -151.0f) return 0.0f;               // below half of the smallest subnormal
    const float e = __builtin_amdgcn_exp2f(t + 64.0f);
    const float v = __builtin_fmaf(e, r * 0.693147182464599609375f, e);
    return v * 5.42101086242752217003726400434970855712890625e-20f;  // 2^-64
  }
  const float e = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(e, r * 0.693147182464599609375f, e);  // e * 2^r, |r| << 1
}

/*! \brief p / s given rcp = 1 / s: one Newton correction on the quotient. The result is
 *  the correctly rounded quotient except for rare half-ulp cases. */
__device__ __forceinline__ float DivideBy(float p, float s, float rcp) {
  const float q = p * rcp;
  const float e = __builtin_fmaf(-q, s, p);
  return __builtin_fmaf(e, rcp, q);
}

template <int THREADS>
__device__ inline float BlockMax(float v, OrderedSumLds<THREADS / kWave> *lds) {
  const int W = THREADS / kWave;
  v = WaveMaxF32(v);
  if (LaneId() == 0) lds->wmax[WaveId()] = v;
  __syncthreads();
  float m = lds->wmax[0];
#pragma unroll
  for (int w = 1; w < W; ++w) {
    const float o = lds->wmax[w];
    m = (m < o) ? o : m;
  }
  return m;
}

/*! \brief THREADS * SLABS * VEC >= cols. VEC == 4 needs 16-byte aligned rows and
 *  cols % 4 == 0. */
template <int THREADS, int SLABS, int VEC>
__global__ void __launch_bounds__(THREADS, 4)  // >= 4 waves per SIMD: two 512-thread rows per CU
    SoftmaxRowKernel(float *dst, int dstride, const float *src, int sstride, int cols) {
  __shared__ OrderedSumLds<THREADS / kWave> lds;
  const int tid = threadIdx.x;
  const float *in = src + static_cast<size_t>(blockIdx.x) * sstride;
  float *out = dst + static_cast<size_t>(blockIdx.x) * dstride;
  const float kNegInf = -__builtin_huge_valf();

  float v[SLABS][VEC];
  float mx = kNegInf;
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int base = (j * THREADS + tid) * VEC;
    if (VEC == 4) {  // cols % 4 == 0: a pack is either whole or absent
      F4 q = {kNegInf, kNegInf, kNegInf, kNegInf};
      if (base < cols) q = StreamLoadF4(in + base);
      v[j][0] = q.x; v[j][1 % VEC] = q.y; v[j][2 % VEC] = q.z; v[j][3 % VEC] = q.w;
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[j][i] = (base + i < cols) ? in[base + i] : kNegInf;
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) mx = (mx < v[j][i]) ? v[j][i] : mx;
  }
  mx = BlockMax<THREADS>(mx, &lds);

#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int base = (j * THREADS + tid) * VEC;
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[j][i] = (base + i < cols) ? ExpNonPositive(v[j][i] - mx) : 0.0f;
  }

  float s = 0.0f;
  int buf = 0;
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    if (j * THREADS * VEC < cols) s = BlockOrderedAdd<THREADS, VEC>(s, v[j], &lds, &buf);
  }

  /* s >= 1 for finite logits (the maximum contributes exp(0)); anything else (NaN or
     infinite logits) takes the plain division so that specials propagate as on the CPU */
  const bool fast_div = s >= 1.0f && s < 3.0e38f;
  const float rcp = 1.0f / s;
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int base = (j * THREADS + tid) * VEC;
    float o[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) o[i] = fast_div ? DivideBy(v[j][i], s, rcp) : v[j][i] / s;
    if (VEC == 4) {
      F4 q;
      q.x = o[0]; q.y = o[1 % VEC]; q.z = o[2 % VEC]; q.w = o[3 % VEC];
      if (base < cols) StreamStoreF4(out + base, q);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        if (base + i < cols) out[base + i] = o[i];
      }
    }
  }
}

/*! \brief any row length: three passes, exp(x - max) parked in dst between them */
template <int THREADS>
__global__ void __launch_bounds__(THREADS)
    SoftmaxLongRowKernel(float *dst, int dstride, const float *src, int sstride, int cols) {
  __shared__ OrderedSumLds<THREADS / kWave> lds;
  const int tid = threadIdx.x;
  const float *in = src + static_cast<size_t>(blockIdx.x) * sstride;
  float *out = dst + static_cast<size_t>(blockIdx.x) * dstride;
  const float kNegInf = -__builtin_huge_valf();
  float mx = kNegInf;
  for (int x = tid; x < cols; x += THREADS) {
    const float e = in[x];
    mx = (mx < e) ? e : mx;
  }
  mx = BlockMax<THREADS>(mx, &lds);
  float s = 0.0f;
  int buf = 0;
  for (int x0 = 0; x0 < cols; x0 += THREADS) {
    const int x = x0 + tid;
    float p[1];
    p[0] = (x < cols) ? ExpNonPositive(in[x] - mx) : 0.0f;
    if (x < cols) out[x] = p[0];
    s = BlockOrderedAdd<THREADS, 1>(s, p, &lds, &buf);
  }
  for (int x = tid; x < cols; x += THREADS) out[x] = out[x] / s;
}

const int kGradBlock = 256;
const int kGradPacks = 2;  // 128-bit packs per thread

/*! \brief grid.x = rows * chunks, a chunk being kGradBlock * kGradPacks * 4 columns.
 *  Consecutive workgroups walk along a row, so the workgroups in flight at any moment
 *  stream one contiguous region of memory. */
template <bool VEC4>
__global__ void __launch_bounds__(kGradBlock)
    SoftmaxGradKernel(float *dst, int dstride, const float *src, int sstride, const float *label,
                      int cols, unsigned chunks) {
  const int y = blockIdx.x / chunks;
  const int chunk = blockIdx.x - y * chunks;
  const int k = static_cast<int>(label[y]);
  const float *in = src + static_cast<size_t>(y) * sstride;
  float *out = dst + static_cast<size_t>(y) * dstride;
  const int chunk0 = chunk * (kGradBlock * kGradPacks * 4);
  if (VEC4) {
    F4 q[kGradPacks];
#pragma unroll
    for (int u = 0; u < kGradPacks; ++u) {
      const int x = chunk0 + (u * kGradBlock + threadIdx.x) * 4;
      if (x + 4 <= cols) q[u] = StreamLoadF4(in + x);
    }
#pragma unroll
    for (int u = 0; u < kGradPacks; ++u) {
      const int x = chunk0 + (u * kGradBlock + threadIdx.x) * 4;
      if (x + 4 <= cols) {
        if (k == x) q[u].x = q[u].x - 1.0f;
        if (k == x + 1) q[u].y = q[u].y - 1.0f;
        if (k == x + 2) q[u].z = q[u].z - 1.0f;
        if (k == x + 3) q[u].w = q[u].w - 1.0f;
        StreamStoreF4(out + x, q[u]);
      } else {
        for (int i = x; i < cols; ++i) out[i] = (i == k) ? in[i] - 1.0f : in[i];
      }
    }
  } else {
#pragma unroll
    for (int u = 0; u < kGradPacks * 4; ++u) {
      const int x = chunk0 + u * kGradBlock + threadIdx.x;
      if (x < cols) out[x] = (x == k) ? in[x] - 1.0f : in[x];
    }
  }
}

}  // namespace mshadow_hipk
#endif  // MSHADOW_AMD_CSRC_SOFTMAX_KERNELS_H_
