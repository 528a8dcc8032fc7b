/*
 * Shared plumbing of the C ABI implementation files: error capture and argument
 * checks. Every exported function is wrapped so that no exception leaves the library
 * and the failure text is kept per thread for mshadow_hip_last_error().
 */
#ifndef MSHADOW_AMD_CSRC_ABI_COMMON_H_
#define MSHADOW_AMD_CSRC_ABI_COMMON_H_

#include <hip/hip_runtime.h>
#include <mshadow_hip.h>

#include <cstdio>
#include <string>

namespace mshadow_abi {

std::string &LastError();

inline int Fail(int code, const std::string &msg) {
  LastError() = msg;
  return code;
}

inline int FromHip(hipError_t e, const char *what) {
  if (e == hipSuccess) return MSHADOW_HIP_OK;
  return Fail(MSHADOW_HIP_ERR_RUNTIME,
              std::string(what) + ": " + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ")");
}

inline hipStream_t AsStream(void *s) { return reinterpret_cast<hipStream_t>(s); }

/* queued-launch check: the reference calls cudaPeekAtLastError after every launch
   (mshadow/cuda/tensor_gpu-inl.cuh:16-21); hipGetLastError also clears the sticky code */
inline int AfterLaunch(const char *what) { return FromHip(hipGetLastError(), what); }

/* looks up, once per device, where the scratch array of the sort that allocates nothing lives
   on the current device (csrc/sort.hip) */
void ResolveSortScratch();

/* compute units of the calling thread's device (looked up once per thread) */
int ComputeUnits();

/* device-to-device copy of a pitched view by the library's own kernel; false: not covered */
bool CopyRowsOnDevice(void *dst, size_t dpitch_bytes, const void *src, size_t spitch_bytes,
                      size_t width_bytes, size_t rows, hipStream_t s);

/* a stream is going away: whatever scratch memory of the library it was given is free again */
void ReleaseReduceScratch(void *stream);
/* looks up, once per device, where the scratch slots of the split reductions live on the current
   device (csrc/ops.hip) */
void ResolveReduceScratch();

}  // namespace mshadow_abi

#define ABI_HIP(call)                                              \
  do {                                                             \
    int st_ = mshadow_abi::FromHip((call), #call);                 \
    if (st_ != MSHADOW_HIP_OK) return st_;                         \
  } while (0)

#define ABI_REQUIRE(cond, msg)                                                        \
  do {                                                                                \
    if (!(cond)) return mshadow_abi::Fail(MSHADOW_HIP_ERR_ARGUMENT,                   \
                                          std::string(__func__) + ": " + (msg));      \
  } while (0)

#endif  // MSHADOW_AMD_CSRC_ABI_COMMON_H_
