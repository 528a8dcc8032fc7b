/*
 * libmshadow_probe - measurement aids for the benchmark harness; no part of the device
 * layer (nothing in libmshadow_hip.so or the headers depends on it).
 *
 *   mshadow_probe_softmax_phases   the register-resident softmax kernel of the library,
 *       compiled here with its time-stamp hook switched on: per row, when each step of the
 *       kernel was reached (100 MHz counter), reduced on the host to mean times per step
 *   mshadow_probe_add_chain        what one dependent float add costs a single wave, with
 *       operands from registers, from LDS (as the column reduction feeds its chain) and
 *       along the lanes (as the softmax row sum adds its list), at a given number of
 *       workgroups, so that the figure can be taken with the whole chip busy
 */
#include <hip/hip_runtime.h>
#include <mshadow_hip.h>
#include "mshadow_hip_probe.h"

#include <algorithm>
#include <functional>
#include <string>
#include <vector>

namespace {
__device__ long long *g_stamps;  //!< [rows][kStampSlots], set before each probe launch
const int kStampSlots = MSHADOW_PROBE_STAMPS;
}  // namespace

#define MSHADOW_ROWSUM_STAMP(step)                                                          \
  {                                                                                         \
    __builtin_amdgcn_sched_barrier(0);                                                      \
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");                             \
    if (threadIdx.x == 0) {                                                                 \
      g_stamps[static_cast<size_t>(blockIdx.x) * kStampSlots + (step)] = wall_clock64();    \
    }                                                                                       \
    __builtin_amdgcn_sched_barrier(0);                                                      \
  }

/* The instrumented kernels are other functions than the library's: in their own namespace,
   or the loader would bind this file's launches to the library's copies of the same names. */
#define mshadow_hipk mshadow_hipk_probe
#include "softmax_kernels.h"

#include <mshadow/hip/kernels/reduce.h>
#define ReduceKeepHighDimSplitKernel ReduceKeepHighDimSplitProbeKernel
#define ReduceKeepHighDimDmaKernel ReduceKeepHighDimDmaProbeKernel
#define ReduceKeepLowestDmaKernel ReduceKeepLowestDmaProbeKernel
#include <mshadow/hip/kernels/reduce_dma.h>
#undef ReduceKeepHighDimSplitKernel
#undef ReduceKeepHighDimDmaKernel
#undef ReduceKeepLowestDmaKernel

#include "abi_common.h"

namespace mshadow_abi {
std::string &LastError() {
  static thread_local std::string text;
  return text;
}
}  // namespace mshadow_abi

using mshadow_abi::AfterLaunch;
using mshadow_abi::AsStream;

namespace {

/*! \brief `iters` rounds of 32 dependent adds whose operand is a register */
__global__ void __launch_bounds__(64) RegisterChainKernel(float *out, float a, int iters) {
  float s = threadIdx.x;
  float addend = a;
  asm volatile("" : "+v"(addend));  // a vector register, as the operand of a real chain is
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int k = 0; k < 32; ++k) {
      s = s + addend;
      asm volatile("" : "+v"(s));
    }
  }
  out[blockIdx.x * 64 + threadIdx.x] = s;
}

/*! \brief the same with binary16 values: one 16-bit add per step, which is what a half_t
 *  `sum += term` amounts to (widen, add in float, round back: one rounding of the exact sum) */
__global__ void __launch_bounds__(64) RegisterChainHalfKernel(float *out, float a, int iters) {
  _Float16 s = static_cast<_Float16>(static_cast<float>(threadIdx.x));
  _Float16 addend = static_cast<_Float16>(a);
  asm volatile("" : "+v"(addend));
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int k = 0; k < 32; ++k) {
      s = s + addend;
      asm volatile("" : "+v"(s));
    }
  }
  out[blockIdx.x * 64 + threadIdx.x] = static_cast<float>(s);
}

/*! \brief the chain of the column reduction: 16 lanes fold `count` floats each from LDS,
 *  four per 128-bit read, the next 32 operands fetched while 32 adds execute */
__global__ void __launch_bounds__(64) LdsChainKernel(float *out, int iters, int count) {
  __shared__ float buf[16 * 1028];
  for (int i = threadIdx.x; i < 16 * 1028; i += 64) buf[i] = i * 1e-3f;
  __syncthreads();
  float s = 0.0f;
  if (threadIdx.x < 16) {
    for (int i = 0; i < iters; ++i) {
      mshadow::hip::ChainFold<mshadow::red::sum, 4>(s, buf + threadIdx.x * 1028, 0, count);
      asm volatile("" : "+v"(s));
    }
  }
  out[blockIdx.x * 64 + threadIdx.x] = s;
}

/*! \brief the chain of the softmax row sum: a sum handed from lane to lane */
__global__ void __launch_bounds__(64) SystolicChainKernel(float *out, float a, int iters) {
  float s = threadIdx.x;
  float addend = a;
  asm volatile("" : "+v"(addend));
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int k = 0; k < 32; ++k) mshadow_hipk::SystolicStep(&s, addend);
  }
  out[blockIdx.x * 64 + threadIdx.x] = s;
}

/*! \brief the memory side of the softmax kernel alone: a workgroup loads its row into
 *  registers exactly as SoftmaxRowKernel does, meets `barriers` workgroup barriers with
 *  `spin` dependent multiply-adds per element in between (a stand-in for the work between
 *  the load and the store), and stores the row */
template <int THREADS, int SLABS>
__global__ void __launch_bounds__(THREADS, 4)
    RowCopyKernel(float *dst, int dstride, const float *src, int sstride, int cols, int barriers,
                  int spin) {
  using mshadow_hipk::F4;
  const int W = THREADS / 64;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane_col = (threadIdx.x & 63) * 4;
  const float *in = src + static_cast<size_t>(blockIdx.x) * sstride;
  float *out = dst + static_cast<size_t>(blockIdx.x) * dstride;
  F4 v[SLABS];
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int c0 = (j * W + wave) * 256;
    v[j] = F4{0.0f, 0.0f, 0.0f, 0.0f};
    if (c0 + static_cast<int>(lane_col) < cols) v[j] = mshadow_hipk::StreamLoadF4(in + c0 + lane_col);
  }
  for (int b = 0; b < barriers; ++b) {
    for (int k = 0; k < spin; ++k) {
#pragma unroll
      for (int j = 0; j < SLABS; ++j) v[j] = v[j] * 1.0000001f + 1e-9f;
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < SLABS; ++j) {
    const int c0 = (j * W + wave) * 256;
    if (c0 + static_cast<int>(lane_col) < cols) mshadow_hipk::StreamStoreF4(out + c0 + lane_col, v[j]);
  }
}


/*! \brief the row copy as a persistent workgroup that is fed from its own next row: while a
 *  row sits in registers (stand-in work, then its stores), the first PRE slabs of the
 *  workgroup's next row are already on their way into LDS by loads that bypass the registers;
 *  the rest of a row (SLABS - PRE slabs) is loaded into registers when the row's turn comes.
 *  A wave reads back from LDS exactly the bytes its own loads delivered, so the hand-over
 *  needs a wait on the wave's own counter and no barrier. The counter retires loads and
 *  stores in issue order: the wait leaves the stores of the row before and the direct
 *  loads of this row outstanding (at most the last slab of either is skipped by a wave);
 *  in front of a workgroup's first row there are no stores to leave. */
template <int THREADS, int SLABS, int PRE>
__global__ void __launch_bounds__(THREADS)
    RowCopyPrefetchKernel(float *dst, int dstride, const float *src, int sstride, int rows, int cols,
                          int barriers, int spin) {
  using mshadow_hipk::F4;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int W = THREADS / 64;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int lane_col = lane * 4;
  unsigned char *mine = lds + static_cast<size_t>(wave) * PRE * 1024;
  auto prefetch = [&](int row) {
    const float *in = src + static_cast<size_t>(row) * sstride;
#pragma unroll
    for (int j = 0; j < PRE; ++j) {
      int col = (j * W + wave) * 256 + lane_col;
      col = col < cols ? col : cols - 4;  // clamped, never consumed
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(in + col),
                                       (__attribute__((address_space(3))) void *)(mine + j * 1024), 16, 0,
                                       2);
    }
  };
  int row = blockIdx.x;
  if (row < rows) prefetch(row);
  for (; row < rows; row += gridDim.x) {
    const float *in = src + static_cast<size_t>(row) * sstride;
    float *out = dst + static_cast<size_t>(row) * dstride;
    F4 v[SLABS];
#pragma unroll
    for (int j = PRE; j < SLABS; ++j) {
      const int c0 = (j * W + wave) * 256;
      v[j] = F4{0.0f, 0.0f, 0.0f, 0.0f};
      if (c0 + lane_col < cols) v[j] = mshadow_hipk::StreamLoadF4(in + c0 + lane_col);
    }
    /* operations issued behind this row's loads into LDS, at least: its own direct loads and,
       from the second row on, the stores of the row before */
    const int kDirect = PRE < SLABS ? SLABS - PRE - 1 : 0;
    const int kLater = (SLABS - 1) + kDirect;
    if (row == static_cast<int>(blockIdx.x)) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kDirect) : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLater) : "memory");
    }
#pragma unroll
    for (int j = 0; j < PRE; ++j) v[j] = *reinterpret_cast<const F4 *>(mine + j * 1024 + lane * 16);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (row + static_cast<int>(gridDim.x) < rows) prefetch(row + gridDim.x);
    for (int b = 0; b < barriers; ++b) {
      for (int k = 0; k < spin; ++k) {
#pragma unroll
        for (int j = 0; j < SLABS; ++j) v[j] = v[j] * 1.0000001f + 1e-9f;
      }
      asm volatile("s_barrier" ::: "memory");
    }
#pragma unroll
    for (int j = 0; j < SLABS; ++j) {
      const int c0 = (j * W + wave) * 256;
      if (c0 + lane_col < cols) mshadow_hipk::StreamStoreF4(out + c0 + lane_col, v[j]);
    }
  }
}

/* Rate of loads into LDS when a workgroup reads `segs` neighbouring segments of `seg_len`
   floats side by side (64 * WIDTH bytes of each in turn), workgroup b taking segments
   b * segs .. b * segs + segs - 1: the pattern of a reduction whose inner chains run one per
   lane over segments that lie one after the other in memory. */
template <int WIDTH>
__global__ void __launch_bounds__(1024) SegRateKernel(const float *src, uint32_t seg_len, uint32_t segs,
                                                      uint32_t piece_instr) {
  const int kRegion = 16 * 64 * WIDTH;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t nwave = blockDim.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  unsigned char *mine = lds + wave * kRegion;
  const int kFloats = WIDTH / 4;
  const uint32_t per_seg = seg_len / (64 * kFloats);          // instructions per segment
  const uint32_t turns = per_seg / piece_instr;               // rounds over the segments
  const uint32_t ninstr = segs * turns * piece_instr / nwave;  // per wave
  const float *base = src + static_cast<size_t>(blockIdx.x) * segs * seg_len + lane * kFloats;
  for (uint32_t i = 0; i + 16 <= ninstr; i += 16) {
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const uint32_t t = (i + q) * nwave + wave;
      /* t counts instructions in the order (turn, segment, instruction of the piece) */
      const uint32_t in_piece = t % piece_instr;
      const uint32_t u = t / piece_instr;
      const uint32_t seg = u % segs, turn = u / segs;
      const size_t at = static_cast<size_t>(seg) * seg_len +
                        static_cast<size_t>(turn * piece_instr + in_piece) * 64 * kFloats;
      const __attribute__((address_space(1))) void *from =
          (const __attribute__((address_space(1))) void *)(base + at);
      __attribute__((address_space(3))) void *to =
          (__attribute__((address_space(3))) void *)(mine + q * 64 * WIDTH);
      if (WIDTH == 4) {
        __builtin_amdgcn_global_load_lds(from, to, 4, 0, 2);
      } else {
        __builtin_amdgcn_global_load_lds(from, to, 16, 0, 2);
      }
    }
    asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

/* Rate of loads from global memory straight into LDS, nothing else: `blockDim.x / 64` waves
   per workgroup issue them in batches of 16 and wait until `window` (16 or 32) are left
   outstanding, so that window .. window + 16 are in flight per wave. WIDTH bytes per
   lane (4 or 16). STRIP == 0: a workgroup reads a contiguous piece of the buffer, an
   instruction 64 * WIDTH consecutive bytes. STRIP > 0: the buffer is a matrix of `rows` x
   `cols` floats, a workgroup reads STRIP columns of every row (what a reduction over the
   rows does), an instruction as many rows as its 64 lanes cover. STRIP == -1: the buffer
   is 64 x gridDim.x segments of equal length, workgroup c reads segments c, c + gridDim.x,
   ... side by side, one instruction's worth of each in turn (what a reduction that keeps
   the second of four dimensions does). */
template <int WIDTH, int STRIP>
__global__ void __launch_bounds__(1024) DmaRateKernel(const float *src, uint32_t stride, uint32_t rows,
                                                      uint32_t cols, int window) {
  const int kRegion = 16 * 64 * WIDTH;   // bytes of LDS a wave cycles through
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t nwave = blockDim.x >> 6;
  const uint32_t lane = threadIdx.x & 63;
  unsigned char *mine = lds + wave * kRegion;
  const int kFloats = WIDTH / 4;
  uint32_t ninstr;
  const float *base;
  size_t step;   // floats between this wave's consecutive instructions
  if (STRIP == 0) {
    const size_t total = static_cast<size_t>(rows) * stride;
    const size_t piece = total / gridDim.x / (64 * kFloats) * (64 * kFloats);
    ninstr = static_cast<uint32_t>(piece / (64 * kFloats)) / nwave;
    base = src + piece * blockIdx.x + (static_cast<size_t>(wave) * 64 + lane) * kFloats;
    step = static_cast<size_t>(nwave) * 64 * kFloats;
  } else if (STRIP == -1) {
    ninstr = 0;
    base = src;
    step = 0;
  } else {
    const int kLanesPerRow = STRIP / kFloats;
    const int kRowsPerInstr = 64 / kLanesPerRow;
    ninstr = rows / kRowsPerInstr / nwave;
    base = src + static_cast<size_t>(wave * kRowsPerInstr + lane / kLanesPerRow) * stride +
           mshadow::hip::StripOfBlock(blockIdx.x, gridDim.x) * STRIP + (lane % kLanesPerRow) * kFloats;
    step = static_cast<size_t>(nwave) * kRowsPerInstr * stride;
  }
  uint32_t seg_len = 0;
  if (STRIP == -1) {
    seg_len = static_cast<uint32_t>(static_cast<size_t>(rows) * stride / 64 / gridDim.x);
    ninstr = 64 * (seg_len / (64 * kFloats)) / nwave;
    base = src + static_cast<size_t>(blockIdx.x) * seg_len + lane * kFloats;
  }
  (void)cols;
  for (uint32_t i = 0; i + 16 <= ninstr; i += 16) {
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      size_t at = (i + q) * step;
      if (STRIP == -1) {
        const uint32_t t = (i + q) * nwave + wave;
        at = static_cast<size_t>(t % 64) * gridDim.x * seg_len + static_cast<size_t>(t / 64) * 64 * kFloats;
      }
      const __attribute__((address_space(1))) void *from =
          (const __attribute__((address_space(1))) void *)(base + at);
      __attribute__((address_space(3))) void *to =
          (__attribute__((address_space(3))) void *)(mine + q * 64 * WIDTH);
      if (WIDTH == 4) {
        __builtin_amdgcn_global_load_lds(from, to, 4, 0, 2);
      } else {
        __builtin_amdgcn_global_load_lds(from, to, 16, 0, 2);
      }
    }
    if (window == 16) {
      asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

/*! \brief a copy by waves that stay: every wave moves `per_wave` pieces of 1 KB (64 lanes x 16
 *  bytes), DEPTH of them on their way at a time. OWN_RUN: the pieces of a wave are one
 *  contiguous run of memory, so the waves resident at any moment read and write as many
 *  separate sequential streams; otherwise piece i of wave w is piece i * waves + w, so that at
 *  any moment the resident waves work side by side on one region. */
template <bool OWN_RUN, int DEPTH>
__global__ void __launch_bounds__(256) StreamCopyKernel(float *dst, const float *src, uint32_t per_wave) {
  using mshadow_hipk::F4;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = blockIdx.x * 4u + (threadIdx.x >> 6);
  const uint32_t waves = gridDim.x * 4u;
  for (uint32_t i = 0; i < per_wave; i += DEPTH) {
    F4 q[DEPTH];
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const size_t piece = OWN_RUN ? static_cast<size_t>(wave) * per_wave + i + u
                                   : static_cast<size_t>(i + u) * waves + wave;
      q[u] = mshadow_hipk::StreamLoadF4(src + piece * 256u + lane * 4u);
    }
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const size_t piece = OWN_RUN ? static_cast<size_t>(wave) * per_wave + i + u
                                   : static_cast<size_t>(i + u) * waves + wave;
      mshadow_hipk::StreamStoreF4(dst + piece * 256u + lane * 4u, q[u]);
    }
  }
}

int TimeKernel(hipStream_t s, float *ms, const std::function<void()> &launch) {
  hipEvent_t a, b;
  ABI_HIP(hipEventCreate(&a));
  ABI_HIP(hipEventCreate(&b));
  launch();  // warm-up
  ABI_HIP(hipStreamSynchronize(s));
  ABI_HIP(hipEventRecord(a, s));
  launch();
  ABI_HIP(hipEventRecord(b, s));
  ABI_HIP(hipEventSynchronize(b));
  ABI_HIP(hipEventElapsedTime(ms, a, b));
  ABI_HIP(hipEventDestroy(a));
  ABI_HIP(hipEventDestroy(b));
  return AfterLaunch("probe kernel");
}

}  // namespace

extern "C" {

const char *mshadow_probe_last_error(void) { return mshadow_abi::LastError().c_str(); }

int mshadow_probe_add_chain(int mode, int workgroups, double *ns_per_add, void *stream) {
  ABI_REQUIRE(ns_per_add != NULL && workgroups >= 1 && workgroups <= 65536, "bad argument");
  hipStream_t s = AsStream(stream);
  float *out = NULL;
  ABI_HIP(hipMalloc(&out, static_cast<size_t>(workgroups) * 64 * sizeof(float)));
  float ms = 0.0f;
  int st;
  double adds;
  if (mode == MSHADOW_PROBE_CHAIN_REGISTER) {
    const int iters = 4096;
    adds = 32.0 * iters;
    st = TimeKernel(s, &ms, [&] {
      hipLaunchKernelGGL(RegisterChainKernel, dim3(workgroups), dim3(64), 0, s, out, 1.5f, iters);
    });
  } else if (mode == MSHADOW_PROBE_CHAIN_REGISTER_F16) {
    const int iters = 4096;
    adds = 32.0 * iters;
    st = TimeKernel(s, &ms, [&] {
      hipLaunchKernelGGL(RegisterChainHalfKernel, dim3(workgroups), dim3(64), 0, s, out, 0.25f, iters);
    });
  } else if (mode == MSHADOW_PROBE_CHAIN_LDS) {
    const int iters = 128, count = 1024;
    adds = static_cast<double>(iters) * count;
    st = TimeKernel(s, &ms, [&] {
      hipLaunchKernelGGL(LdsChainKernel, dim3(workgroups), dim3(64), 0, s, out, iters, count);
    });
  } else if (mode == MSHADOW_PROBE_CHAIN_LANES) {
    const int iters = 4096;
    adds = 32.0 * iters;
    st = TimeKernel(s, &ms, [&] {
      hipLaunchKernelGGL(SystolicChainKernel, dim3(workgroups), dim3(64), 0, s, out, 1.5f, iters);
    });
  } else {
    (void)hipFree(out);
    ABI_REQUIRE(false, "unknown mode");
  }
  (void)hipFree(out);
  if (st != MSHADOW_HIP_OK) return st;
  *ns_per_add = static_cast<double>(ms) * 1e6 / adds;
  return MSHADOW_HIP_OK;
}

int mshadow_probe_row_copy(float *dst, int dstride, const float *src, int sstride, int rows,
                           int cols, int barriers, int spin, int resident, double *kernel_us,
                           void *stream) {
  ABI_REQUIRE(resident == 1 || resident == 2, "one or two rows resident per CU");
  ABI_REQUIRE(rows >= 1 && cols > 16384 && cols <= 32768 && cols % 4 == 0 && sstride % 4 == 0 &&
                  dstride % 4 == 0 && kernel_us != NULL, "16384 < cols <= 32768, rows of whole packs");
  hipStream_t s = AsStream(stream);
  float ms = 0.0f;
  const int st = TimeKernel(s, &ms, [&] {
    /* one row per CU: dynamic LDS the kernel never touches keeps a second workgroup off the CU */
    hipLaunchKernelGGL((RowCopyKernel<512, 16>), dim3(rows), dim3(512), resident == 1 ? 90000 : 0, s, dst,
                       dstride, src, sstride, cols, barriers, spin);
  });
  if (st != MSHADOW_HIP_OK) return st;
  *kernel_us = ms * 1e3;
  return MSHADOW_HIP_OK;
}

int mshadow_probe_row_copy_prefetch(float *dst, int dstride, const float *src, int sstride, int rows,
                                    int cols, int threads, int prefetch_slabs, int barriers, int spin,
                                    int workgroups, double *kernel_us, void *stream) {
  ABI_REQUIRE(rows >= 1 && cols > 28672 && cols <= 32768 && cols % 4 == 0 && sstride % 4 == 0 &&
                  dstride % 4 == 0 && kernel_us != NULL, "28672 < cols <= 32768, rows of whole packs");
  ABI_REQUIRE(workgroups >= 1 && workgroups <= rows, "1..rows workgroups");
  ABI_REQUIRE(reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0,
              "16-byte aligned");
  hipStream_t s = AsStream(stream);
  float ms = 0.0f;
  int st = MSHADOW_HIP_ERR_ARGUMENT;
#define PROBE_PREFETCH(T, SL, PRE)                                                                  \
  if (threads == T && prefetch_slabs == PRE) {                                                      \
    const size_t lds = static_cast<size_t>(T) / 64 * PRE * 1024;                                    \
    ABI_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&RowCopyPrefetchKernel<T, SL, PRE>), \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));           \
    st = TimeKernel(s, &ms, [&] {                                                                   \
      hipLaunchKernelGGL((RowCopyPrefetchKernel<T, SL, PRE>), dim3(workgroups), dim3(T), lds, s, dst, \
                         dstride, src, sstride, rows, cols, barriers, spin);                        \
    });                                                                                             \
  }
  PROBE_PREFETCH(1024, 8, 8)
  PROBE_PREFETCH(1024, 8, 4)
  PROBE_PREFETCH(512, 16, 8)
  PROBE_PREFETCH(512, 16, 4)
  PROBE_PREFETCH(512, 16, 16)
#undef PROBE_PREFETCH
  ABI_REQUIRE(st != MSHADOW_HIP_ERR_ARGUMENT, "threads / prefetch_slabs: 1024 with 8 or 4, 512 with 16, 8 or 4");
  if (st != MSHADOW_HIP_OK) return st;
  *kernel_us = ms * 1e3;
  return MSHADOW_HIP_OK;
}

int mshadow_probe_seg_rate(const float *src, size_t floats, int seg_len, int nseg, int segs, int width,
                           int waves, int piece_instr, double *kernel_us, void *stream) {
  ABI_REQUIRE(src != NULL && kernel_us != NULL && seg_len >= 64 && nseg >= 1 && segs >= 1, "bad argument");
  ABI_REQUIRE(static_cast<size_t>(seg_len) * nseg <= floats && nseg % segs == 0, "segments beyond the buffer");
  ABI_REQUIRE((width == 4 || width == 16) && waves >= 1 && waves <= 16 && piece_instr >= 1, "bad argument");
  ABI_REQUIRE(seg_len % 4 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0, "16-byte aligned segments");
  hipStream_t s = AsStream(stream);
  const size_t lds = static_cast<size_t>(waves) * 16 * 64 * width;
  float ms = 0.0f;
  int st;
  if (width == 4) {
    st = TimeKernel(s, &ms, [&] {
      hipLaunchKernelGGL((SegRateKernel<4>), dim3(nseg / segs), dim3(waves * 64), lds, s, src,
                         static_cast<uint32_t>(seg_len), static_cast<uint32_t>(segs),
                         static_cast<uint32_t>(piece_instr));
    });
  } else {
    ABI_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&SegRateKernel<16>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    st = TimeKernel(s, &ms, [&] {
      hipLaunchKernelGGL((SegRateKernel<16>), dim3(nseg / segs), dim3(waves * 64), lds, s, src,
                         static_cast<uint32_t>(seg_len), static_cast<uint32_t>(segs),
                         static_cast<uint32_t>(piece_instr));
    });
  }
  if (st != MSHADOW_HIP_OK) return st;
  *kernel_us = ms * 1e3;
  return MSHADOW_HIP_OK;
}

int mshadow_probe_highdim_split(float *dst, const float *warm, const float *src, int n, int c, int y,
                                int x, int config, double *kernel_us, void *stream) {
  using namespace mshadow::hip;
  ABI_REQUIRE(dst != NULL && warm != NULL && src != NULL && kernel_us != NULL, "NULL argument");
  ABI_REQUIRE(n >= 1 && c >= 1 && (static_cast<long long>(y) * x) % 4 == 0 && y * x >= 4, "segments of whole packs");
  hipStream_t s = AsStream(stream);
  uint32_t *scratch = NULL;
  const size_t words = static_cast<size_t>(n) * c;
  ABI_HIP(hipMalloc(&scratch, (words + kSplitCounterWords) * 4));
  ABI_HIP(hipMemsetAsync(scratch, 0, (words + kSplitCounterWords) * 4, s));
  uint32_t *counter = scratch + words;
  const uint32_t seg = static_cast<uint32_t>(y) * x;
  const mshadow::FastDivU32 div_seg(seg), div_x(static_cast<uint32_t>(x));
  hipEvent_t a, b;
  ABI_HIP(hipEventCreate(&a));
  ABI_HIP(hipEventCreate(&b));
  typedef mshadow::sv::saveto SV;
  typedef mshadow::red::sum RD;
  auto launch = [&](const float *from) {
#define PROBE_SPLIT(ID, SEGS, LOADERS, SLOTS, W)                                                    \
  if (config == ID) {                                                                               \
    typedef SplitRing<SEGS, LOADERS, SLOTS, W> Ring;                                                \
    hipLaunchKernelGGL((ReduceKeepHighDimSplitProbeKernel<SV, RD, float, Ring>),                    \
                       dim3((n * c + SEGS - 1) / SEGS), dim3(Ring::kThreads), 0, s, dst, from, seg, \
                       static_cast<uint32_t>(n), static_cast<uint32_t>(c), 1u, seg, div_seg, 1.0f,  \
                       scratch, counter);                                                           \
  }
    PROBE_SPLIT(0, 64, 8, 8, 4)
    PROBE_SPLIT(1, 32, 8, 8, 4)
    PROBE_SPLIT(2, 16, 8, 4, 16)
    PROBE_SPLIT(3, 32, 8, 4, 16)
    PROBE_SPLIT(4, 16, 4, 8, 4)
    PROBE_SPLIT(5, 32, 8, 6, 4)
    PROBE_SPLIT(6, 64, 8, 6, 4)
    PROBE_SPLIT(7, 32, 4, 8, 4)
    PROBE_SPLIT(8, 16, 8, 8, 4)
#undef PROBE_SPLIT
    if (config < 0) {
      hipLaunchKernelGGL((ReduceKeepHighDimDmaProbeKernel<SV, RD, float, 64>), dim3(c), dim3(kDmaThreads), 0,
                         s, dst, from, static_cast<uint32_t>(x), static_cast<uint32_t>(n),
                         static_cast<uint32_t>(c), static_cast<uint32_t>(y), static_cast<uint32_t>(x),
                         div_x, 1.0f);
    }
  };
  launch(src);
  launch(warm);   // what the timed launch reads is no longer in the memory-side cache
  ABI_HIP(hipEventRecord(a, s));
  launch(src);
  ABI_HIP(hipEventRecord(b, s));
  ABI_HIP(hipEventSynchronize(b));
  float ms = 0.0f;
  ABI_HIP(hipEventElapsedTime(&ms, a, b));
  ABI_HIP(hipEventDestroy(a));
  ABI_HIP(hipEventDestroy(b));
  ABI_HIP(hipFree(scratch));
  *kernel_us = ms * 1e3;
  return AfterLaunch("probe kernel");
}

int mshadow_probe_softmax_phases(float *dst, int dstride, const float *src, int sstride, int rows,
                                 int cols, int variant, double *mean_us, double *resident_us,
                                 double *kernel_us, int *fallback_rows, void *stream) {
  ABI_REQUIRE(variant >= 0 && variant <= 3, "variant 0 to 3");
  ABI_REQUIRE(rows >= 1 && cols > 16384 && cols <= 32768 && cols % 4 == 0 && sstride % 4 == 0 &&
                  dstride % 4 == 0, "the probe covers the 512-thread, 16-slab kernel: 16384 < cols <= 32768, rows of whole packs");
  ABI_REQUIRE(mean_us != NULL && resident_us != NULL && kernel_us != NULL && fallback_rows != NULL,
              "NULL result");
  hipStream_t s = AsStream(stream);
  long long *stamps = NULL;
  const size_t n = static_cast<size_t>(rows) * kStampSlots;
  ABI_HIP(hipMalloc(&stamps, n * sizeof(long long)));
  ABI_HIP(hipMemsetAsync(stamps, 0, n * sizeof(long long), s));
  ABI_HIP(hipMemcpyToSymbolAsync(HIP_SYMBOL(g_stamps), &stamps, sizeof(stamps), 0,
                                 hipMemcpyHostToDevice, s));
  float ms = 0.0f;
  const int st = TimeKernel(s, &ms, [&] {
    if (variant == 0) {
      hipLaunchKernelGGL((mshadow_hipk::SoftmaxRowKernel<512, 16, 4, false>), dim3(rows), dim3(512), 0,
                         s, dst, dstride, src, sstride, cols);
    } else if (variant == 1) {  // one row per CU: LDS the kernel never touches keeps a second one off
      hipLaunchKernelGGL((mshadow_hipk::SoftmaxRowKernel<512, 16, 4, false>), dim3(rows), dim3(512),
                         90000, s, dst, dstride, src, sstride, cols);
    } else if (variant == 2) {  // one row per CU, on sixteen waves
      hipLaunchKernelGGL((mshadow_hipk::SoftmaxRowKernel<1024, 8, 4, false>), dim3(rows), dim3(1024),
                         90000, s, dst, dstride, src, sstride, cols);
    } else {  // three rows per CU, four waves each (a wave per SIMD, 168 registers)
      hipLaunchKernelGGL((mshadow_hipk::SoftmaxRowKernel<256, 32, 4, false, 3>), dim3(rows), dim3(256),
                         0, s, dst, dstride, src, sstride, cols);
    }
  });
  if (st != MSHADOW_HIP_OK) {
    (void)hipFree(stamps);
    return st;
  }
  *kernel_us = ms * 1e3;
  std::vector<long long> h(n);
  ABI_HIP(hipMemcpy(h.data(), stamps, n * sizeof(long long), hipMemcpyDeviceToHost));
  ABI_HIP(hipFree(stamps));
  /* the steps a row passed through, in the order of the kernel; a step a row did not
     reach (the fall-back) has no stamp and is left out of that row's chain of intervals */
  static const int order[] = MSHADOW_PROBE_STAMP_ORDER;
  const int norder = static_cast<int>(sizeof(order) / sizeof(order[0]));
  std::vector<double> sum(kStampSlots, 0.0);
  std::vector<long> cnt(kStampSlots, 0);
  double resident = 0.0;
  *fallback_rows = 0;
  for (int r = 0; r < rows; ++r) {
    const long long *t = &h[static_cast<size_t>(r) * kStampSlots];
    if (t[MSHADOW_PROBE_STAMP_FALLBACK] != 0) ++*fallback_rows;
    long long prev = t[order[0]];
    for (int i = 1; i < norder; ++i) {
      const long long now = t[order[i]];
      if (now == 0) continue;
      sum[order[i]] += static_cast<double>(now - prev);
      ++cnt[order[i]];
      prev = now;
    }
    resident += static_cast<double>(prev - t[order[0]]);
  }
  for (int i = 0; i < kStampSlots; ++i) mean_us[i] = cnt[i] ? sum[i] / cnt[i] / 100.0 : -1.0;
  mean_us[order[0]] = 0.0;
  *resident_us = resident / rows / 100.0;
  return MSHADOW_HIP_OK;
}

int mshadow_probe_dma_rate(const float *src, int sstride, int rows, int cols, int strip, int width,
                           int waves, int window, double *kernel_us, void *stream) {
  ABI_REQUIRE(src != NULL && kernel_us != NULL && rows >= 1024 && cols >= 64 && sstride >= cols,
              "a matrix of at least 1024 x 64");
  ABI_REQUIRE(waves >= 1 && waves <= 16, "1..16 waves");
  ABI_REQUIRE(window == 16 || window == 32, "16 or 32 loads left outstanding");
  ABI_REQUIRE((width == 4 || width == 16) &&
                  (strip == -1 || strip == 0 || strip == 16 || strip == 32 || strip == 64),
              "width 4 or 16 bytes, strip -1, 0, 16, 32 or 64");
  ABI_REQUIRE(cols % 64 == 0 && sstride % 4 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0,
              "rows of whole strips, 16-byte aligned");
  hipStream_t s = AsStream(stream);
  const unsigned grid = strip == 0 ? 1024u : strip == -1 ? 256u : static_cast<unsigned>(cols / strip);
  const size_t lds = static_cast<size_t>(waves) * 16 * 64 * width;
  ABI_REQUIRE(lds <= 160 * 1024, "too many waves for the LDS");
  float ms = 0.0f;
  int st;
#define PROBE_DMA(W, S)                                                                       \
  {                                                                                           \
    ABI_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&DmaRateKernel<W, S>),         \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));     \
    st = TimeKernel(s, &ms, [&] {                                                             \
      hipLaunchKernelGGL((DmaRateKernel<W, S>), dim3(grid), dim3(waves * 64), lds, s, src,    \
                         static_cast<uint32_t>(sstride), static_cast<uint32_t>(rows),         \
                         static_cast<uint32_t>(cols), window);                                \
    });                                                                                       \
  }
  if (width == 4 && strip == -1) PROBE_DMA(4, -1)
  else if (width == 16 && strip == -1) PROBE_DMA(16, -1)
  else if (width == 4 && strip == 0) PROBE_DMA(4, 0)
  else if (width == 16 && strip == 0) PROBE_DMA(16, 0)
  else if (width == 4 && strip == 16) PROBE_DMA(4, 16)
  else if (width == 16 && strip == 16) PROBE_DMA(16, 16)
  else if (width == 4 && strip == 32) PROBE_DMA(4, 32)
  else if (width == 16 && strip == 32) PROBE_DMA(16, 32)
  else if (width == 4 && strip == 64) PROBE_DMA(4, 64)
  else PROBE_DMA(16, 64)
#undef PROBE_DMA
  if (st != MSHADOW_HIP_OK) return st;
  *kernel_us = ms * 1e3;
  return MSHADOW_HIP_OK;
}

int mshadow_probe_stream_copy(float *dst, const float *src, size_t floats, int workgroups, int own_run,
                              double *kernel_us, void *stream) {
  ABI_REQUIRE(dst != NULL && src != NULL && kernel_us != NULL && workgroups >= 1, "bad argument");
  const size_t waves = static_cast<size_t>(workgroups) * 4;
  const int kDepth = 4;
  ABI_REQUIRE(floats % (waves * 256 * kDepth) == 0 && floats / (waves * 256) < (1ull << 31),
              "floats must be a multiple of workgroups x 4 KB x 4");
  const uint32_t per_wave = static_cast<uint32_t>(floats / (waves * 256));
  hipStream_t s = AsStream(stream);
  float ms = 0.0f;
  const int st = TimeKernel(s, &ms, [&] {
    if (own_run) {
      hipLaunchKernelGGL((StreamCopyKernel<true, kDepth>), dim3(workgroups), dim3(256), 0, s, dst, src, per_wave);
    } else {
      hipLaunchKernelGGL((StreamCopyKernel<false, kDepth>), dim3(workgroups), dim3(256), 0, s, dst, src, per_wave);
    }
  });
  if (st != MSHADOW_HIP_OK) return st;
  *kernel_us = ms * 1e3;
  return MSHADOW_HIP_OK;
}

}  // extern "C"
