/*
 * libmshadow_hip - C ABI of the gfx950 (MI355X) device layer behind mshadow's
 * Tensor<gpu> / Stream<gpu> API.
 *
 * The reference has no FFI: its GPU device is a set of C++ templates that call the
 * CUDA runtime and launch CUDA kernels (mshadow/tensor_gpu-inl.h,
 * mshadow/stream_gpu-inl.h, mshadow/cuda/tensor_gpu-inl.cuh). This header is the
 * boundary that replaces those call sites. Each entry names the reference code it
 * stands in for. Three groups:
 *   1. runtime      device, stream, event, memory, copy
 *   2. launch       start a kernel instantiated in the caller's translation unit
 *                   (expression templates compile there, not in this library)
 *   3. fixed ops    whole operations on plain (pointer, pitch, shape) arguments
 *
 * Conventions: every function returns 0 on success and a non-zero code otherwise,
 * with a thread-local message available from mshadow_hip_last_error(); no exception
 * crosses the boundary. Pointers are device pointers unless named host. `stream` is
 * the opaque handle from mshadow_hip_stream_create, or NULL for the device's default
 * stream. Pitches ("stride") are in ELEMENTS, as in mshadow's Tensor::stride_; sizes
 * and indices are 32-bit like mshadow's index_t. Kernels are asynchronous: a call
 * returns once the work is queued on `stream`. The library never allocates device
 * memory on its own; the caller owns every buffer.
 */
#ifndef MSHADOW_HIP_H_
#define MSHADOW_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MSHADOW_HIP_ABI_VERSION 1

/* status codes */
enum {
  MSHADOW_HIP_OK = 0,
  MSHADOW_HIP_ERR_RUNTIME = 1,  /* a HIP runtime call failed; text in last_error */
  MSHADOW_HIP_ERR_ARGUMENT = 2, /* shapes / pointers / enums rejected before launch */
  MSHADOW_HIP_ERR_UNSUPPORTED = 3
};

/* saver: how a result is combined into dst (mshadow/base.h:539-602, sv::) */
enum { MSHADOW_HIP_SAVETO = 0, MSHADOW_HIP_PLUSTO = 1, MSHADOW_HIP_MINUSTO = 2,
       MSHADOW_HIP_MULTO = 3, MSHADOW_HIP_DIVTO = 4 };
/* reducer (mshadow/base.h:604-862, red::) */
enum { MSHADOW_HIP_SUM = 0, MSHADOW_HIP_MAX = 1, MSHADOW_HIP_MIN = 2 };
/* copy direction for mshadow_hip_memcpy2d_async */
enum { MSHADOW_HIP_H2D = 1, MSHADOW_HIP_D2H = 2, MSHADOW_HIP_D2D = 3, MSHADOW_HIP_H2H = 0 };

/* message of the last failure on the calling thread ("" if none) */
const char *mshadow_hip_last_error(void);
int mshadow_hip_abi_version(void);

/* ------------------------------------------------------------------ 1. runtime */

typedef struct mshadow_hip_props {
  char name[256];
  char arch[64];             /* e.g. "gfx950:sramecc+:xnack-" */
  int compute_units;
  int wavefront_size;
  int max_threads_per_block;
  int clock_khz;
  int memory_clock_khz;
  int memory_bus_bits;
  int l2_bytes;
  size_t lds_bytes_per_block;
  size_t total_global_mem;
} mshadow_hip_props;

/* InitTensorEngine<gpu> / SetDevice<gpu>: mshadow/tensor_gpu-inl.h:14-36
   (cudaGetDeviceCount, cudaSetDevice, cudaGetDeviceProperties) */
int mshadow_hip_device_count(int *count);
int mshadow_hip_set_device(int device);
int mshadow_hip_get_device(int *device);
int mshadow_hip_get_props(int device, mshadow_hip_props *out);
int mshadow_hip_device_sync(void);

/* Stream<gpu>: mshadow/stream_gpu-inl.h:61-74 (Wait, CheckIdle), :181-211
   (NewStream / DeleteStream -> cudaStreamCreate / cudaStreamDestroy) */
int mshadow_hip_stream_create(void **stream);
int mshadow_hip_stream_destroy(void *stream);
int mshadow_hip_stream_sync(void *stream);
int mshadow_hip_stream_query(void *stream, int *idle);

/* timing (the reference has none; used by the benchmark harness) */
int mshadow_hip_event_create(void **event);
int mshadow_hip_event_destroy(void *event);
int mshadow_hip_event_record(void *event, void *stream);
int mshadow_hip_event_sync(void *event);
int mshadow_hip_event_elapsed_ms(void *start, void *stop, float *ms);

/* A sequence of launches recorded once and replayed (the reference has nothing of the kind: it
   launches kernel by kernel). Everything queued on `stream` between begin and end - launches of
   this library and of kernels compiled with the caller alike - is recorded instead of run;
   end hands back an executable graph that mshadow_hip_graph_launch queues on any stream of the
   same device as often as wanted, with the pointers and shapes of the recording. While a stream
   records, only launches and copies between device buffers may be queued on it: no allocation,
   no synchronisation, no copy from or to pageable host memory, and none of the entry points
   that allocate or wait (the sort entries, mshadow_hip_blas_*). `stream` must not be NULL. */
int mshadow_hip_graph_begin(void *stream);
int mshadow_hip_graph_end(void *stream, void **graph);
int mshadow_hip_graph_launch(void *graph, void *stream);
int mshadow_hip_graph_destroy(void *graph);

/* AllocSpace / FreeSpace<gpu>: mshadow/tensor_gpu-inl.h:37-56 (cudaMallocPitch,
   cudaFree). pitch_bytes is a multiple of 256 when rows > 1. */
int mshadow_hip_malloc_pitch(void **ptr, size_t *pitch_bytes, size_t width_bytes, size_t rows);
int mshadow_hip_malloc(void **ptr, size_t bytes);
int mshadow_hip_free(void *ptr);
/* AllocHost_ / FreeHost_<gpu>: mshadow/tensor_cpu-inl.h:58-69 (pinned host memory) */
int mshadow_hip_malloc_host(void **host_ptr, size_t bytes);
int mshadow_hip_free_host(void *host_ptr);
/* Copy cpu<->gpu, gpu<->gpu: mshadow/tensor_gpu-inl.h:57-92 (cudaMemcpy2DAsync).
   Pitches and width in BYTES here, like the runtime call it replaces. Device to device the
   copy is a kernel of this library (streaming 128-bit or 32-bit accesses, any number of
   bytes) when addresses, width and pitches are multiples of 4 bytes, the runtime's copy
   otherwise; the two views must not overlap. */
int mshadow_hip_memcpy2d_async(void *dst, size_t dpitch_bytes, const void *src,
                               size_t spitch_bytes, size_t width_bytes, size_t rows, int kind,
                               void *stream);
int mshadow_hip_memset_async(void *dst, int byte_value, size_t bytes, void *stream);
/* dst = scalar on a (rows, cols) view of 32-bit elements with pitch dstride (elements):
   what `tensor = value` and NewTensor's initial value do through MapExp in the reference
   (mshadow/tensor_gpu-inl.h:101-116 with a ScalarExp source). `bits` is the element's
   bit pattern. A kernel, not a memset: it may be recorded into a graph. No limit on the
   element count short of `int` rows and columns (runs of rows of less than 2^31 elements
   each are launched one after the other). */
int mshadow_hip_fill_32(void *dst, int dstride, int rows, int cols, uint32_t bits, void *stream);
/* The runs of whole rows mshadow_hip_fill_32 launches for a (rows, cols) view (wide != 0: rows
   of 128-bit packs): first row and row count of up to max_runs runs into runs[2 i], runs[2 i + 1];
   returns their number. Host arithmetic only - no launch, no device - so that the splitting can
   be checked for shapes too large to allocate. No counterpart in the reference. */
int mshadow_hip_fill_32_runs(int rows, int cols, int wide, int64_t *runs, int max_runs);

/* ------------------------------------------------------------------ 2. launch */

/* The <<<grid, block, lds, stream>>> launch plus cudaPeekAtLastError of
   mshadow/cuda/tensor_gpu-inl.cuh:16-21 and :95-120: `kernel` is the host-side
   address of a __global__ function compiled by hipcc in the caller's own
   translation unit (an instantiation of the kernel templates shipped in
   mshadow/hip/); `args` is the array of pointers to its arguments. */
int mshadow_hip_launch(const void *kernel, const uint32_t grid[3], const uint32_t block[3],
                       void **args, size_t lds_bytes, void *stream);
int mshadow_hip_peek_last_error(void);
/* Grid size for `work_items` items at `items_per_block` per block: enough blocks to
   cover the work, capped at `max_waves` resident rounds of the device's CUs
   (replaces the kBaseGridNum / kMaxGridNum heuristics of tensor_gpu-inl.cuh:25-45). */
int mshadow_hip_suggest_grid(size_t work_items, size_t items_per_block, int max_waves,
                             uint32_t *grid_x);

/* ------------------------------------------------------------------ 3. fixed ops */

/* Softmax(dst, energy): mshadow/tensor_gpu-inl.h:157-161 -> cuda::Softmax,
   tensor_gpu-inl.cuh:330-393. Row-wise; dst may alias src. The row sum is taken in
   the CPU path's left-to-right order (tensor_cpu-inl.h:277-281). */
int mshadow_hip_softmax_f32(float *dst, int dstride, const float *src, int sstride, int rows,
                            int cols, void *stream);
/* The row-sum stage of Softmax on its own: sums[r] = the float32 sum of the cols
   non-negative terms of row r added left to right into one accumulator, exactly as the
   loop at mshadow/tensor_cpu-inl.h:277-281 accumulates exp(energy - max). Runs the same
   device code as mshadow_hip_softmax_f32 (rows of any length) and exists so that
   this stage can be compared bit for bit with a serial sum, which the full operation
   does not allow because the device exponential differs from libm's. */
int mshadow_hip_softmax_rowsum_f32(float *sums, const float *terms, int tstride, int rows,
                                   int cols, void *stream);
/* SoftmaxGrad(dst, src, label): mshadow/tensor_gpu-inl.h:169-174 ->
   tensor_gpu-inl.cuh:239-256, :395-412. label holds `rows` floats, truncated to int. */
int mshadow_hip_softmax_grad_f32(float *dst, int dstride, const float *src, int sstride,
                                 const float *label, int rows, int cols, void *stream);

/* The gradient family in one entry: SoftmaxGrad with ignore_label and SmoothSoftmaxGrad with
   and without it, mshadow/tensor_gpu-inl.h:176-199 -> tensor_gpu-inl.cuh:258-328, 414-477
   (CPU definitions tensor_cpu-inl.h:304-362). flags: MSHADOW_HIP_GRAD_SMOOTH uses alpha
   (label entry: src - 1 + alpha, others: src - alpha / (cols - 1)); MSHADOW_HIP_GRAD_IGNORE
   zeroes the rows whose label equals ignore_label (both truncated to int). flags = 0 is
   mshadow_hip_softmax_grad_f32. */
#define MSHADOW_HIP_GRAD_SMOOTH 1
#define MSHADOW_HIP_GRAD_IGNORE 2
int mshadow_hip_softmax_grad_ex_f32(float *dst, int dstride, const float *src, int sstride,
                                    const float *label, int rows, int cols, int flags,
                                    float ignore_label, float alpha, void *stream);
/* Softmax on 3-D tensors (d0, d1, d2), over the middle dimension, row pitch on d2:
   mshadow/tensor_gpu-inl.h:163-167 -> tensor_gpu-inl.cuh:479-524 (CPU tensor_cpu-inl.h:474-495). */
int mshadow_hip_softmax3d_f32(float *dst, int dstride, const float *src, int sstride, int d0,
                              int d1, int d2, void *stream);
/* SoftmaxGrad / SmoothSoftmaxGrad on 3-D tensors, label (d0, d2) with pitch lstride:
   mshadow/tensor_gpu-inl.h:201-214 -> tensor_gpu-inl.cuh:526-597 (CPU tensor_cpu-inl.h:364-462). */
int mshadow_hip_softmax3d_grad_f32(float *dst, int dstride, const float *src, int sstride,
                                   const float *label, int lstride, int d0, int d1, int d2,
                                   int flags, float ignore_label, float alpha, void *stream);
/* AddTakeGrad(dst, index, src): dst[clamp(index[y], 0, k_rows - 1)] += src[y] for y in order
   (mshadow/tensor_gpu-inl.h:216-222 -> tensor_gpu-inl.cuh:599-672; CPU tensor_cpu-inl.h:497-508).
   index holds n_index entries of int32 (index_is_int != 0) or float. Rows that are named
   several times receive their additions in index order, as on the CPU. */
int mshadow_hip_add_take_grad_f32(float *dst, int dstride, int k_rows, const void *index,
                                  int index_is_int, int n_index, const float *src, int sstride,
                                  int cols, void *stream);
/* AddTakeGradLargeBatch(dst, sorted, index, src): dst[sorted[y]] += src[index[y]] for y in
   order (mshadow/tensor_gpu-inl.h:224-232 -> tensor_gpu-inl.cuh:674-760; CPU
   tensor_cpu-inl.h:510-518). Needs no workspace here. */
int mshadow_hip_add_take_grad_large_batch_f32(float *dst, int dstride, int k_rows,
                                              const void *sorted, const void *index,
                                              int index_is_int, int n_index, const float *src,
                                              int sstride, int cols, void *stream);
/* IndexFill(dst, index, src): dst[index[y]] = src[y]; the last entry naming a row counts
   (mshadow/tensor_gpu-inl.h:234-240 -> tensor_gpu-inl.cuh:762-782; CPU tensor_cpu-inl.h:520-528). */
int mshadow_hip_index_fill_f32(float *dst, int dstride, int k_rows, const void *index,
                               int index_is_int, int n_index, const float *src, int sstride,
                               int cols, void *stream);

/* Random<gpu>::GetRandInt / SampleUniform / SampleGaussian (mshadow/random.h:372-568, cuRAND
   there): Philox-4x32-10 blocks of four words; element e of a call uses block `counter + e / 4`
   of the stream (seed, subsequence), word e % 4. The generator has no state in memory: the
   caller advances `counter` by (elements + 3) / 4 per call. Uniform values lie strictly inside
   (a, b) up to rounding; normal values are mu + z * sigma with z from Box-Muller. The values
   are not cuRAND's. dstride in elements. */
int mshadow_hip_random_u32(uint32_t *dst, size_t n, uint64_t seed, uint64_t subsequence,
                           uint64_t counter, void *stream);
int mshadow_hip_random_uniform_f32(float *dst, int dstride, int rows, int cols, uint64_t seed,
                                   uint64_t subsequence, uint64_t counter, float a, float b,
                                   void *stream);
int mshadow_hip_random_normal_f32(float *dst, int dstride, int rows, int cols, uint64_t seed,
                                  uint64_t subsequence, uint64_t counter, float mu, float sigma,
                                  void *stream);
/* The same for Random<gpu, double> (mshadow/random.h:486-514: curandGenerateUniformDouble /
   curandGenerateNormalDouble there). A value takes two words, 52 bits of them: element e of a
   call uses block `counter + e / 2`, words 2 (e % 2) and 2 (e % 2) + 1; the caller advances
   `counter` by (elements + 1) / 2 per call. Box-Muller runs in double on the block's two
   uniforms. */
int mshadow_hip_random_uniform_f64(double *dst, int dstride, int rows, int cols, uint64_t seed,
                                   uint64_t subsequence, uint64_t counter, double a, double b,
                                   void *stream);
int mshadow_hip_random_normal_f64(double *dst, int dstride, int rows, int cols, uint64_t seed,
                                  uint64_t subsequence, uint64_t counter, double mu, double sigma,
                                  void *stream);

/* dst = transpose(src, axes) / dst = swapaxis<a1, a2>(src) on dense tensors of 32-bit
   elements: dst axis i is src axis axes[i]; `shape` is the source's, ndim <= 6
   (mshadow/extension/transpose.h:24-88, swapaxis.h:20-106, evaluated there element by element
   through the generic map kernel). dst and src must not overlap. */
int mshadow_hip_permute_32(void *dst, const void *src, int ndim, const int *shape,
                           const int *axes, void *stream);

/* SortByKey(keys, values, is_ascend): stable sort of the pairs by key, in place
   (mshadow/tensor_gpu-inl.h:231-235 -> tensor_gpu-inl.cuh:784-806, thrust::stable_sort_by_key;
   CPU tensor_cpu-inl.h:531-559). Keys and values are 32-bit elements; key_kind says how the key
   bits are ordered; values are moved as opaque words. Pairs of equivalent keys (+0.0f and
   -0.0f are equivalent) keep their order in both directions. The scratch memory is the
   caller's: `workspace` holds at least the number of bytes the first call reports for n and
   is 256-byte aligned. VectorizedSort(values, segments) of the reference
   (tensor_cpu-inl.h:561-566) is two of these calls. */
#define MSHADOW_HIP_KEY_F32 0
#define MSHADOW_HIP_KEY_I32 1
#define MSHADOW_HIP_KEY_U32 2
int mshadow_hip_sort_by_key_workspace(size_t n, size_t *bytes);
int mshadow_hip_sort_by_key_32(void *keys, int key_kind, void *values, size_t n, int is_ascend,
                               void *workspace, size_t workspace_bytes, void *stream);
/* The same sort for callers that cannot allocate device memory (serving loops, harnesses
   that forbid it). It has no counterpart in the reference. The scratch memory is an array
   inside the library, one copy per GPU (about 40 MiB, held from the library's load until the
   process ends); the call itself allocates and frees nothing. Where the array lives on a GPU
   is looked up when mshadow_hip_set_device selects that GPU (else on the first call there);
   a call then consists of a host-side size query and three kernel launches. It has not been
   exercised under graph capture.
   At most MSHADOW_HIP_SORT_NOALLOC_MAX pairs; more is an argument error. Every call on a GPU
   uses that GPU's one array: calls that overlap in time on the same GPU (different streams
   or host threads) race on it and must be ordered by the caller. */
#define MSHADOW_HIP_SORT_NOALLOC_MAX (1u << 20)
int mshadow_hip_sort_by_key_32_noalloc(void *keys, int key_kind, void *values, size_t n,
                                       int is_ascend, void *stream);

/* MapReduceKeepLowest<Saver, Reducer>(dst, src, scale): mshadow/tensor_gpu-inl.h:118-133
   -> MapRedKeepLowestKernel, tensor_gpu-inl.cuh:122-168. dst[x] <saver>= scale *
   reduce_y src[y][x], rows >= 1, reduced top to bottom like tensor_cpu-inl.h:221-227. */
int mshadow_hip_reduce_keep_lowest_f32(float *dst, const float *src, int sstride, int rows,
                                       int cols, int reducer, int saver, float scale,
                                       void *stream);
/* MapReduceKeepHighDim<Saver, Reducer, dimkeep>: mshadow/tensor_gpu-inl.h:135-156 ->
   MapReduceKeepDim1Kernel, tensor_gpu-inl.cuh:170-215, on the equivalent 4-D view
   (n, c, y, x) with row pitch sstride: dst[c] <saver>= scale * reduce_n(reduce_{y,x}
   src[n][c][y][x]) in the two-level order of tensor_cpu-inl.h:254-267. */
int mshadow_hip_reduce_keep_highdim_f32(float *dst, const float *src, int sstride, int n, int c,
                                        int y, int x, int reducer, int saver, float scale,
                                        void *stream);
/* Scratch memory for a reduction kernel that spreads the inner (n, c) chains of
   MapReduceKeepHighDim over more workgroups than there are kept indices (the reference's
   kernel, tensor_gpu-inl.cuh:170-215, runs one block per kept index and needs none): `words`
   32-bit words for the inner results and a block of counters that are zero between launches
   (what the kernel template expects: mshadow/hip/kernels/reduce_dma.h), both inside
   a device array that is part of the library (nothing is allocated). One slot per stream and
   GPU, returned again on every call with that stream until mshadow_hip_stream_destroy; launches
   that use it must be queued on that stream. *partial == NULL: none to be had (more words than
   a slot holds, or every slot of the GPU taken) - the caller then runs a kernel that needs
   none. Called by mshadow_hip_reduce_keep_highdim_f32 itself and by the header API for the
   element types whose kernels are instantiated with the caller. */
int mshadow_hip_reduce_scratch(void *stream, size_t words, uint32_t **partial, uint32_t **counter);

/* dst = pool<Reducer>(src, Shape2(ph, pw), ky, kx, sy, sx): the MapPlanKernel launch of
   tensor_gpu-inl.cuh:67-120 with Plan<PoolingExp>::Eval (extension/spatial_pool.h:125-142)
   as its body. src is planes x h x w with row pitch sstride, dst planes x ph x pw. */
int mshadow_hip_pool_f32(float *dst, int dstride, const float *src, int sstride, int planes,
                         int h, int w, int ph, int pw, int ky, int kx, int sy, int sx,
                         int reducer, void *stream);
/* dst = unpool<Reducer>(src, pooled, grad, ky, kx, sy, sx): same launch with
   Plan<UnPoolingExp>::Eval (extension/spatial_unpool.h:102-125). */
int mshadow_hip_unpool_f32(float *dst, int dstride, const float *src, int sstride,
                           const float *pooled, int pstride, const float *grad, int gstride,
                           int planes, int h, int w, int ph, int pw, int ky, int kx, int sy,
                           int sx, int reducer, void *stream);

/* col = unpack_patch2col(pad(img, pad_y, pad_x), ky, kx, sy, sx, dy, dx): MapPlanKernel
   with Plan<UnpackPatchToColXExp>::Eval (extension/unpack_patch2col.h:126-141) over
   Plan<PaddingExp>::Eval (extension/pad.h:87-99). img is (n, c, h, w) with row pitch
   istride; col is (ky*kx*c) x (oh*ow*n) with row pitch cstride. f16 = raw binary16 bits. */
int mshadow_hip_im2col_f16(uint16_t *col, int cstride, const uint16_t *img, int istride, int n,
                           int c, int h, int w, int ky, int kx, int sy, int sx, int dy, int dx,
                           int pad_y, int pad_x, void *stream);
int mshadow_hip_im2col_f32(float *col, int cstride, const float *img, int istride, int n, int c,
                           int h, int w, int ky, int kx, int sy, int sx, int dy, int dx,
                           int pad_y, int pad_x, void *stream);
/* img = crop(pack_col2patch(col, (n, c, h+2*pad_y, w+2*pad_x), ky, kx, sy, sx, dy, dx),
   (h, w), pad_y, pad_x): MapPlanKernel with Plan<CroppingExp>::Eval (extension/crop.h:
   103-110) over Plan<PackColToPatchXExp>::Eval (extension/pack_col2patch.h:118-144);
   overlapping patches are added in (py, px) order in the element type. */
int mshadow_hip_col2im_f16(uint16_t *img, int istride, const uint16_t *col, int cstride, int n,
                           int c, int h, int w, int ky, int kx, int sy, int sx, int dy, int dx,
                           int pad_y, int pad_x, void *stream);
int mshadow_hip_col2im_f32(float *img, int istride, const float *col, int cstride, int n, int c,
                           int h, int w, int ky, int kx, int sy, int sx, int dy, int dx,
                           int pad_y, int pad_x, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MSHADOW_HIP_H_ */
