/*
 * SortByKey on the device: a stable sort of (key, value) pairs by key, in place.
 *
 * The reference sorts with thrust::stable_sort_by_key under less<> / greater<>
 * (mshadow/cuda/tensor_gpu-inl.cuh:784-806); its CPU path is std::stable_sort of an index
 * vector under keys[i1] < keys[i2] resp. > (mshadow/tensor_cpu-inl.h:531-559). Both define
 * the result completely: pairs ordered by key, pairs of equivalent keys in their original
 * order - in either direction - where +0.0f and -0.0f are equivalent.
 *
 * Here: every key is mapped to a 32-bit unsigned rank word whose unsigned order is the
 * requested order (sign-flip for floats and signed integers, -0.0f folded onto +0.0f,
 * complemented for descending), paired with its position; the (rank, position) pairs go
 * through rocPRIM's radix sort, which is stable, so equivalent keys stay in position order;
 * keys and values are then gathered by position from copies taken before the sort. All
 * scratch memory comes from the caller (mshadow_hip_sort_by_key_workspace tells how much).
 * Keys that are NaN have no place in the reference's ordering (its comparator is not a
 * strict weak order on them); here they sort after every number when ascending.
 */
#include <cstring>
#include <mutex>

#include <rocprim/device/device_radix_sort.hpp>

#include "./abi_common.h"

using mshadow_abi::AfterLaunch;
using mshadow_abi::AsStream;

namespace {

const int kSortBlock = 256;

__device__ __forceinline__ uint32_t RankWord(uint32_t bits, int key_kind, bool ascend) {
  uint32_t r = bits;
  if (key_kind == MSHADOW_HIP_KEY_F32) {
    if (bits == 0x80000000u) r = bits = 0u;  // -0.0f and +0.0f are equivalent keys
    r = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
  } else if (key_kind == MSHADOW_HIP_KEY_I32) {
    r = bits ^ 0x80000000u;
  }
  return ascend ? r : ~r;
}

/*! \brief rank words and positions for the sort, and copies of the pairs for the gather */
__global__ void __launch_bounds__(kSortBlock)
    SortPrepareKernel(const uint32_t *keys, const uint32_t *values, uint32_t n, int key_kind,
                      bool ascend, uint32_t *rank, uint32_t *pos, uint32_t *key_copy,
                      uint32_t *value_copy) {
  const uint32_t i = blockIdx.x * kSortBlock + threadIdx.x;
  if (i >= n) return;
  const uint32_t k = keys[i];
  rank[i] = RankWord(k, key_kind, ascend);
  pos[i] = i;
  key_copy[i] = k;
  value_copy[i] = values[i];
}

__global__ void __launch_bounds__(kSortBlock)
    SortGatherKernel(uint32_t *keys, uint32_t *values, uint32_t n, const uint32_t *pos,
                     const uint32_t *key_copy, const uint32_t *value_copy) {
  const uint32_t i = blockIdx.x * kSortBlock + threadIdx.x;
  if (i >= n) return;
  const uint32_t from = pos[i];
  keys[i] = key_copy[from];
  values[i] = value_copy[from];
}

/*! \brief the six arrays of n words at the front of the workspace, 256-byte aligned each */
struct SortLayout {
  size_t array_bytes;
  size_t arrays_total;
  explicit SortLayout(size_t n) {
    array_bytes = (n * sizeof(uint32_t) + 255) / 256 * 256;
    arrays_total = 6 * array_bytes;
  }
};

int RadixTempBytes(size_t n, size_t *bytes) {
  uint32_t *none = NULL;
  *bytes = 0;
  return mshadow_abi::FromHip(
      rocprim::radix_sort_pairs(NULL, *bytes, none, none, none, none, n, 0, 32, hipStream_t(0)),
      "radix sort (size query)");
}

/*! \brief the sort proper, with every scratch array carved out of `base` (256-byte aligned,
 *  at least SortLayout(n).arrays_total + temp bytes); shared by both entry points */
int SortInWorkspace(void *keys, int key_kind, void *values, size_t n, int is_ascend, char *base,
                    size_t temp, void *stream) {
  int st;
  const SortLayout lay(n);
  uint32_t *rank_in = reinterpret_cast<uint32_t *>(base + 0 * lay.array_bytes);
  uint32_t *rank_out = reinterpret_cast<uint32_t *>(base + 1 * lay.array_bytes);
  uint32_t *pos_in = reinterpret_cast<uint32_t *>(base + 2 * lay.array_bytes);
  uint32_t *pos_out = reinterpret_cast<uint32_t *>(base + 3 * lay.array_bytes);
  uint32_t *key_copy = reinterpret_cast<uint32_t *>(base + 4 * lay.array_bytes);
  uint32_t *value_copy = reinterpret_cast<uint32_t *>(base + 5 * lay.array_bytes);
  void *radix_temp = base + lay.arrays_total;
  hipStream_t s = AsStream(stream);
  const uint32_t count = static_cast<uint32_t>(n);
  const unsigned grid = (count + kSortBlock - 1) / kSortBlock;
  hipLaunchKernelGGL(SortPrepareKernel, dim3(grid), dim3(kSortBlock), 0, s,
                     static_cast<const uint32_t *>(keys), static_cast<const uint32_t *>(values),
                     count, key_kind, is_ascend != 0, rank_in, pos_in, key_copy, value_copy);
  st = AfterLaunch("sort_by_key (prepare)");
  if (st != MSHADOW_HIP_OK) return st;
  ABI_HIP(rocprim::radix_sort_pairs(radix_temp, temp, rank_in, rank_out, pos_in, pos_out, n, 0, 32,
                                    s));
  hipLaunchKernelGGL(SortGatherKernel, dim3(grid), dim3(kSortBlock), 0, s,
                     static_cast<uint32_t *>(keys), static_cast<uint32_t *>(values), count,
                     pos_out, key_copy, value_copy);
  return AfterLaunch("sort_by_key (gather)");
}

/* ---- the scratch memory of mshadow_hip_sort_by_key_32_noalloc ----
 * One array per GPU, part of the library's code object: it exists from the moment the
 * library is loaded on a device until the process ends, so the entry point never asks the
 * runtime for memory. Its layout is the one SortInWorkspace carves out of a caller's
 * workspace: six arrays of n words, then rocPRIM's temporary storage. */
const size_t kNoAllocMaxPairs = MSHADOW_HIP_SORT_NOALLOC_MAX;
const size_t kNoAllocRadixTempMax = 16u << 20;  // rocPRIM asks for about 8 n bytes + tables
const size_t kScratchBytes = 6 * kNoAllocMaxPairs * sizeof(uint32_t) + kNoAllocRadixTempMax;

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

/* `scratch` names a host-side stand-in in host code, not device memory. The address of each
   device's copy is asked from the runtime once, with that device current, and kept here;
   host code only ever uses these addresses. */
const int kMaxDevices = 64;
std::mutex g_scratch_mutex;
char *g_scratch_ptr[kMaxDevices] = {NULL};

int ScratchOfCurrentDevice(char **ptr) {
  int dev = -1;
  int st = mshadow_abi::FromHip(hipGetDevice(&dev), "hipGetDevice");
  if (st != MSHADOW_HIP_OK) return st;
  if (dev < 0 || dev >= kMaxDevices) {
    return mshadow_abi::Fail(MSHADOW_HIP_ERR_UNSUPPORTED, "device ordinal beyond the scratch table");
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == NULL) {
    void *p = NULL;
    st = mshadow_abi::FromHip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)),
                              "hipGetSymbolAddress(scratch)");
    if (st != MSHADOW_HIP_OK) return st;
    if (p == NULL || reinterpret_cast<uintptr_t>(p) % 256 != 0) {
      return mshadow_abi::Fail(MSHADOW_HIP_ERR_RUNTIME, "scratch array has no aligned device address");
    }
    g_scratch_ptr[dev] = static_cast<char *>(p);
  }
  *ptr = g_scratch_ptr[dev];
  return MSHADOW_HIP_OK;
}

}  // namespace

namespace mshadow_abi {
/* called when a device is selected (mshadow_hip_set_device): the runtime's lookup of the
   scratch array on that device - loading the code object there, if need be - happens then and
   not inside the first sort */
void ResolveSortScratch() {
  char *unused = NULL;
  if (ScratchOfCurrentDevice(&unused) != MSHADOW_HIP_OK) (void)hipGetLastError();
}
}  // namespace mshadow_abi

extern "C" {

int mshadow_hip_sort_by_key_workspace(size_t n, size_t *bytes) {
  ABI_REQUIRE(bytes != NULL, "NULL result pointer");
  ABI_REQUIRE(n < (1ull << 31), "too many elements");
  *bytes = 0;
  if (n == 0) return MSHADOW_HIP_OK;
  size_t temp = 0;
  const int st = RadixTempBytes(n, &temp);
  if (st != MSHADOW_HIP_OK) return st;
  *bytes = SortLayout(n).arrays_total + (temp + 255) / 256 * 256;
  return MSHADOW_HIP_OK;
}

int mshadow_hip_sort_by_key_32(void *keys, int key_kind, void *values, size_t n, int is_ascend,
                               void *workspace, size_t workspace_bytes, void *stream) {
  ABI_REQUIRE(key_kind == MSHADOW_HIP_KEY_F32 || key_kind == MSHADOW_HIP_KEY_I32 ||
                  key_kind == MSHADOW_HIP_KEY_U32, "unknown key kind");
  ABI_REQUIRE(n < (1ull << 31), "too many elements");
  if (n == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(keys != NULL && values != NULL, "NULL tensor");
  ABI_REQUIRE(workspace != NULL, "NULL workspace");
  ABI_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 256 == 0, "workspace must be 256-byte aligned");
  size_t temp = 0;
  int st = RadixTempBytes(n, &temp);
  if (st != MSHADOW_HIP_OK) return st;
  ABI_REQUIRE(workspace_bytes >= SortLayout(n).arrays_total + temp,
              "workspace smaller than mshadow_hip_sort_by_key_workspace reports");
  return SortInWorkspace(keys, key_kind, values, n, is_ascend, static_cast<char *>(workspace),
                         temp, stream);
}

int mshadow_hip_sort_by_key_32_noalloc(void *keys, int key_kind, void *values, size_t n,
                                       int is_ascend, void *stream) {
  ABI_REQUIRE(key_kind == MSHADOW_HIP_KEY_F32 || key_kind == MSHADOW_HIP_KEY_I32 ||
                  key_kind == MSHADOW_HIP_KEY_U32, "unknown key kind");
  ABI_REQUIRE(n <= kNoAllocMaxPairs,
              "more pairs than MSHADOW_HIP_SORT_NOALLOC_MAX; use mshadow_hip_sort_by_key_32 "
              "with a workspace of the caller");
  if (n == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(keys != NULL && values != NULL, "NULL tensor");
  size_t temp = 0;
  int st = RadixTempBytes(n, &temp);
  if (st != MSHADOW_HIP_OK) return st;
  ABI_REQUIRE(SortLayout(n).arrays_total + temp <= kScratchBytes,
              "the radix sort asks for more temporary storage than the scratch array holds");
  char *base = NULL;
  st = ScratchOfCurrentDevice(&base);
  if (st != MSHADOW_HIP_OK) return st;
  /* Nothing in the scratch memory has to start at zero: the prepare kernel writes the four
     arrays the sort reads, the sort writes its outputs and initialises its own temporary
     storage on the stream, and the gather reads only what those wrote. */
  return SortInWorkspace(keys, key_kind, values, n, is_ascend, base, temp, stream);
}

}  // extern "C"
