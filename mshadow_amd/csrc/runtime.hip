/*
 * C ABI, groups 1 and 2: device / stream / event / memory / copy and the generic
 * kernel launch. Thin, stateless wrappers over the HIP runtime (copies between device
 * tensors run a kernel of the library where alignment allows); see
 * include/mshadow_hip.h for the contract of each entry point.
 */
#include "abi_common.h"

#include <cstring>

namespace mshadow_abi {
std::string &LastError() {
  static thread_local std::string msg;
  return msg;
}
}  // namespace mshadow_abi

namespace mshadow_abi {
int ComputeUnits() {
  static thread_local int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) {
      cus = p.multiProcessorCount;
    } else {
      (void)hipGetLastError();
      cus = 256;  // MI355X
    }
  }
  return cus;
}
}  // namespace mshadow_abi

using namespace mshadow_abi;

extern "C" {

const char *mshadow_hip_last_error(void) { return LastError().c_str(); }
int mshadow_hip_abi_version(void) { return MSHADOW_HIP_ABI_VERSION; }

int mshadow_hip_device_count(int *count) {
  ABI_REQUIRE(count != NULL, "count is NULL");
  *count = 0;
  hipError_t e = hipGetDeviceCount(count);
  if (e == hipErrorNoDevice) {
    *count = 0;
    (void)hipGetLastError();
    return MSHADOW_HIP_OK;
  }
  return FromHip(e, "hipGetDeviceCount");
}
int mshadow_hip_set_device(int device) {
  ABI_HIP(hipSetDevice(device));
  ResolveSortScratch();
  ResolveReduceScratch();
  return MSHADOW_HIP_OK;
}
int mshadow_hip_get_device(int *device) {
  ABI_REQUIRE(device != NULL, "device is NULL");
  ABI_HIP(hipGetDevice(device));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_get_props(int device, mshadow_hip_props *out) {
  ABI_REQUIRE(out != NULL, "out is NULL");
  hipDeviceProp_t p;
  ABI_HIP(hipGetDeviceProperties(&p, device));
  memset(out, 0, sizeof(*out));
  snprintf(out->name, sizeof(out->name), "%s", p.name);
  snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
  out->compute_units = p.multiProcessorCount;
  out->wavefront_size = p.warpSize;
  out->max_threads_per_block = p.maxThreadsPerBlock;
  out->clock_khz = p.clockRate;
  out->memory_clock_khz = p.memoryClockRate;
  out->memory_bus_bits = p.memoryBusWidth;
  out->l2_bytes = p.l2CacheSize;
  out->lds_bytes_per_block = p.sharedMemPerBlock;
  out->total_global_mem = p.totalGlobalMem;
  return MSHADOW_HIP_OK;
}
int mshadow_hip_device_sync(void) {
  ABI_HIP(hipDeviceSynchronize());
  return MSHADOW_HIP_OK;
}

int mshadow_hip_stream_create(void **stream) {
  ABI_REQUIRE(stream != NULL, "stream is NULL");
  hipStream_t s;
  ABI_HIP(hipStreamCreate(&s));  // default priority: streams of mixed priority are avoided
  *stream = s;
  return MSHADOW_HIP_OK;
}
int mshadow_hip_stream_destroy(void *stream) {
  if (stream == NULL) return MSHADOW_HIP_OK;
  ReleaseReduceScratch(stream);
  ABI_HIP(hipStreamDestroy(AsStream(stream)));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_stream_sync(void *stream) {
  ABI_HIP(hipStreamSynchronize(AsStream(stream)));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_stream_query(void *stream, int *idle) {
  ABI_REQUIRE(idle != NULL, "idle is NULL");
  hipError_t e = hipStreamQuery(AsStream(stream));
  if (e == hipErrorNotReady) {
    *idle = 0;
    (void)hipGetLastError();
    return MSHADOW_HIP_OK;
  }
  *idle = 1;
  return FromHip(e, "hipStreamQuery");
}

int mshadow_hip_graph_begin(void *stream) {
  ABI_REQUIRE(stream != NULL, "the default stream cannot record");
  ABI_HIP(hipStreamBeginCapture(AsStream(stream), hipStreamCaptureModeThreadLocal));
  return MSHADOW_HIP_OK;
}

int mshadow_hip_graph_end(void *stream, void **graph) {
  ABI_REQUIRE(stream != NULL && graph != NULL, "NULL stream or result");
  *graph = NULL;
  hipGraph_t recorded = NULL;
  ABI_HIP(hipStreamEndCapture(AsStream(stream), &recorded));
  ABI_REQUIRE(recorded != NULL, "nothing was recorded");
  hipGraphExec_t exec = NULL;
  const hipError_t e = hipGraphInstantiate(&exec, recorded, NULL, NULL, 0);
  (void)hipGraphDestroy(recorded);
  ABI_HIP(e);
  *graph = exec;
  return MSHADOW_HIP_OK;
}

int mshadow_hip_graph_launch(void *graph, void *stream) {
  ABI_REQUIRE(graph != NULL, "NULL graph");
  ABI_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), AsStream(stream)));
  return MSHADOW_HIP_OK;
}

int mshadow_hip_graph_destroy(void *graph) {
  if (graph == NULL) return MSHADOW_HIP_OK;
  ABI_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph)));
  return MSHADOW_HIP_OK;
}

int mshadow_hip_event_create(void **event) {
  ABI_REQUIRE(event != NULL, "event is NULL");
  hipEvent_t e;
  ABI_HIP(hipEventCreate(&e));
  *event = e;
  return MSHADOW_HIP_OK;
}
int mshadow_hip_event_destroy(void *event) {
  if (event == NULL) return MSHADOW_HIP_OK;
  ABI_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_event_record(void *event, void *stream) {
  ABI_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), AsStream(stream)));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_event_sync(void *event) {
  ABI_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_event_elapsed_ms(void *start, void *stop, float *ms) {
  ABI_REQUIRE(ms != NULL, "ms is NULL");
  ABI_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                              reinterpret_cast<hipEvent_t>(stop)));
  return MSHADOW_HIP_OK;
}

int mshadow_hip_malloc_pitch(void **ptr, size_t *pitch_bytes, size_t width_bytes, size_t rows) {
  ABI_REQUIRE(ptr != NULL && pitch_bytes != NULL, "output pointer is NULL");
  /* 256-byte pitch: every row starts on a full 128-bit-access and cache-line boundary.
     A single row keeps its natural width (the contiguous case of AllocSpace). */
  size_t pitch = width_bytes;
  if (rows > 1) pitch = (width_bytes + 255) / 256 * 256;
  size_t total = pitch * (rows ? rows : 1);
  if (total == 0) total = 256;
  ABI_HIP(hipMalloc(ptr, total));
  *pitch_bytes = pitch;
  return MSHADOW_HIP_OK;
}
int mshadow_hip_malloc(void **ptr, size_t bytes) {
  ABI_REQUIRE(ptr != NULL, "ptr is NULL");
  ABI_HIP(hipMalloc(ptr, bytes ? bytes : 256));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_free(void *ptr) {
  if (ptr == NULL) return MSHADOW_HIP_OK;
  ABI_HIP(hipFree(ptr));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_malloc_host(void **host_ptr, size_t bytes) {
  ABI_REQUIRE(host_ptr != NULL, "host_ptr is NULL");
  ABI_HIP(hipHostMalloc(host_ptr, bytes ? bytes : 256, hipHostMallocPortable));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_free_host(void *host_ptr) {
  if (host_ptr == NULL) return MSHADOW_HIP_OK;
  ABI_HIP(hipHostFree(host_ptr));
  return MSHADOW_HIP_OK;
}
int mshadow_hip_memcpy2d_async(void *dst, size_t dpitch_bytes, const void *src,
                               size_t spitch_bytes, size_t width_bytes, size_t rows, int kind,
                               void *stream) {
  hipMemcpyKind k;
  switch (kind) {
    case MSHADOW_HIP_H2D: k = hipMemcpyHostToDevice; break;
    case MSHADOW_HIP_D2H: k = hipMemcpyDeviceToHost; break;
    case MSHADOW_HIP_D2D: k = hipMemcpyDeviceToDevice; break;
    case MSHADOW_HIP_H2H: k = hipMemcpyHostToHost; break;
    default: return Fail(MSHADOW_HIP_ERR_ARGUMENT, "mshadow_hip_memcpy2d_async: bad kind");
  }
  if (width_bytes == 0 || rows == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(dst != NULL && src != NULL, "NULL buffer");
  ABI_REQUIRE(dpitch_bytes >= width_bytes && spitch_bytes >= width_bytes, "pitch < width");
  if (kind == MSHADOW_HIP_D2D &&
      CopyRowsOnDevice(dst, dpitch_bytes, src, spitch_bytes, width_bytes, rows, AsStream(stream))) {
    return AfterLaunch("copy");
  }
  if (dpitch_bytes == width_bytes && spitch_bytes == width_bytes) {
    ABI_HIP(hipMemcpyAsync(dst, src, width_bytes * rows, k, AsStream(stream)));
  } else {
    ABI_HIP(hipMemcpy2DAsync(dst, dpitch_bytes, src, spitch_bytes, width_bytes, rows, k,
                             AsStream(stream)));
  }
  return MSHADOW_HIP_OK;
}
int mshadow_hip_memset_async(void *dst, int byte_value, size_t bytes, void *stream) {
  if (bytes == 0) return MSHADOW_HIP_OK;
  ABI_HIP(hipMemsetAsync(dst, byte_value, bytes, AsStream(stream)));
  return MSHADOW_HIP_OK;
}

int mshadow_hip_launch(const void *kernel, const uint32_t grid[3], const uint32_t block[3],
                       void **args, size_t lds_bytes, void *stream) {
  ABI_REQUIRE(kernel != NULL && grid != NULL && block != NULL, "NULL argument");
  ABI_REQUIRE(grid[0] > 0 && grid[1] > 0 && grid[2] > 0, "empty grid");
  ABI_REQUIRE(block[0] * block[1] * block[2] > 0 && block[0] * block[1] * block[2] <= 1024,
              "block size out of range");
  ABI_REQUIRE(lds_bytes <= 160 * 1024, "more than 160 KB of LDS requested");
  ABI_HIP(hipLaunchKernel(kernel, dim3(grid[0], grid[1], grid[2]),
                          dim3(block[0], block[1], block[2]), args, lds_bytes, AsStream(stream)));
  return AfterLaunch("kernel launch");
}
int mshadow_hip_peek_last_error(void) { return FromHip(hipPeekAtLastError(), "pending error"); }

int mshadow_hip_suggest_grid(size_t work_items, size_t items_per_block, int max_waves,
                             uint32_t *grid_x) {
  ABI_REQUIRE(grid_x != NULL && items_per_block > 0, "bad argument");
  const int cus = ComputeUnits();
  size_t blocks = (work_items + items_per_block - 1) / items_per_block;
  if (blocks == 0) blocks = 1;
  /* a 256-thread block holds 4 waves; 8 such blocks fill a CU's 32 wave slots */
  const size_t cap = static_cast<size_t>(cus) * 8 * (max_waves > 0 ? max_waves : 1);
  if (blocks > cap) blocks = cap;
  *grid_x = static_cast<uint32_t>(blocks);
  return MSHADOW_HIP_OK;
}

}  // extern "C"
