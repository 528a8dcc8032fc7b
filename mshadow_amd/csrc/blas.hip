/*
 * Dense linear algebra of the C ABI: GEMM / GEMV / GER / DOT forwarded to rocBLAS.
 *
 * These are the calls BLASEngine<gpu, DType> of the reference makes into cuBLAS
 * (mshadow/dot_engine-inl.h:501-838). They are plain library routines, so nothing here is
 * a kernel of this backend; the work of this file is the plumbing around them:
 *  - rocBLAS is opened with dlopen on the first call, so the library has no load-time
 *    dependency on it and the elementwise / reduction paths never pay for it;
 *  - one rocBLAS handle per (host thread, device), created on first use and kept for the
 *    life of the process; every call binds it to the caller's stream first, which is what
 *    BLASEngine::SetStream does in the reference (:610-614);
 *  - batched problems use the strided-batched routines (the reference builds pointer arrays
 *    in a caller-provided workspace for cuBLAS < 8 and uses the strided form from 8 on,
 *    :626-668).
 */
#include <dlfcn.h>
#include <mshadow_hip_blas.h>
#include <rocblas/rocblas.h>

#include <map>
#include <mutex>

#include "./abi_common.h"

using mshadow_abi::AsStream;
using mshadow_abi::Fail;

namespace {

/*! \brief the rocBLAS entry points this file uses, resolved once */
struct RocBlasApi {
#define MSHADOW_ROCBLAS_FUNCTIONS(X) \
  X(rocblas_create_handle)           \
  X(rocblas_set_stream)              \
  X(rocblas_set_pointer_mode)        \
  X(rocblas_status_to_string)        \
  X(rocblas_gemm_strided_batched_ex) \
  X(rocblas_sgemv_strided_batched)   \
  X(rocblas_dgemv_strided_batched)   \
  X(rocblas_sger_strided_batched)    \
  X(rocblas_dger_strided_batched)    \
  X(rocblas_sdot)                    \
  X(rocblas_ddot)
#define MSHADOW_DECLARE(name) decltype(&::name) name = nullptr;
  MSHADOW_ROCBLAS_FUNCTIONS(MSHADOW_DECLARE)
#undef MSHADOW_DECLARE
  std::string error;  // why the library could not be used, empty when it can
  bool ok = false;

  RocBlasApi() {
    const char *names[] = {"librocblas.so.5", "librocblas.so"};
    void *lib = nullptr;
    for (const char *n : names) {
      lib = dlopen(n, RTLD_NOW | RTLD_LOCAL);
      if (lib != nullptr) break;
    }
    if (lib == nullptr) {
      const char *why = dlerror();
      error = std::string("rocBLAS could not be loaded: ") + (why ? why : "unknown reason");
      return;
    }
#define MSHADOW_RESOLVE(name)                                            \
  name = reinterpret_cast<decltype(name)>(dlsym(lib, #name));            \
  if (name == nullptr) {                                                 \
    error = std::string("rocBLAS has no symbol ") + #name;               \
    return;                                                              \
  }
    MSHADOW_ROCBLAS_FUNCTIONS(MSHADOW_RESOLVE)
#undef MSHADOW_RESOLVE
#undef MSHADOW_ROCBLAS_FUNCTIONS
    ok = true;
  }
};

const RocBlasApi &Api() {
  static const RocBlasApi api;  // initialised once, thread-safe
  return api;
}

int FromRocBlas(rocblas_status st, const char *what) {
  if (st == rocblas_status_success) return MSHADOW_HIP_OK;
  return Fail(MSHADOW_HIP_ERR_RUNTIME,
              std::string(what) + ": " + Api().rocblas_status_to_string(st));
}

/*! \brief the calling thread's handle for the current device, bound to `stream` */
int HandleFor(void *stream, rocblas_handle *out) {
  const RocBlasApi &api = Api();
  if (!api.ok) return Fail(MSHADOW_HIP_ERR_UNSUPPORTED, api.error);
  int device = 0;
  int st = mshadow_abi::FromHip(hipGetDevice(&device), "hipGetDevice");
  if (st != MSHADOW_HIP_OK) return st;
  /* handles are never destroyed: at thread or process exit the runtime they belong to may
     already be gone */
  static thread_local std::map<int, rocblas_handle> *handles = new std::map<int, rocblas_handle>();
  auto it = handles->find(device);
  if (it == handles->end()) {
    rocblas_handle h = nullptr;
    st = FromRocBlas(api.rocblas_create_handle(&h), "rocblas_create_handle");
    if (st != MSHADOW_HIP_OK) return st;
    it = handles->insert(std::make_pair(device, h)).first;
  }
  st = FromRocBlas(api.rocblas_set_stream(it->second, AsStream(stream)), "rocblas_set_stream");
  if (st != MSHADOW_HIP_OK) return st;
  *out = it->second;
  return MSHADOW_HIP_OK;
}

inline rocblas_operation Op(int trans) {
  return trans ? rocblas_operation_transpose : rocblas_operation_none;
}

/*! \brief rows x cols of a stored operand that is read as `trans ? cols x rows : rows x cols` */
inline bool LeadingOk(int ld, int rows) { return ld >= (rows > 1 ? rows : 1); }

inline bool BatchOk(int batch, long long sa, long long sb, long long sc) {
  return batch >= 0 && sa >= 0 && sb >= 0 && sc >= 0;
}

}  // namespace

extern "C" {

int mshadow_hip_blas_gemm(int dtype, int transa, int transb, int m, int n, int k, double alpha,
                          const void *A, int lda, long long stride_a, const void *B, int ldb,
                          long long stride_b, double beta, void *C, int ldc, long long stride_c,
                          int batch, void *stream) {
  ABI_REQUIRE(dtype == MSHADOW_HIP_BLAS_F32 || dtype == MSHADOW_HIP_BLAS_F64 ||
                  dtype == MSHADOW_HIP_BLAS_F16,
              "unknown element type");
  ABI_REQUIRE(m >= 0 && n >= 0 && k >= 0, "negative dimension");
  ABI_REQUIRE(BatchOk(batch, stride_a, stride_b, stride_c), "negative batch count or stride");
  ABI_REQUIRE(LeadingOk(lda, transa ? k : m), "lda is smaller than the rows of A as stored");
  ABI_REQUIRE(LeadingOk(ldb, transb ? n : k), "ldb is smaller than the rows of B as stored");
  ABI_REQUIRE(LeadingOk(ldc, m), "ldc is smaller than m");
  if (m == 0 || n == 0 || batch == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(C != nullptr && (k == 0 || (A != nullptr && B != nullptr)), "null operand");
  ABI_REQUIRE(batch == 1 || stride_c >= static_cast<long long>(ldc) * n,
              "the results of a batch overlap");
  rocblas_handle h;
  int st = HandleFor(stream, &h);
  if (st != MSHADOW_HIP_OK) return st;
  const float alpha_f = static_cast<float>(alpha), beta_f = static_cast<float>(beta);
  const void *pa = &alpha_f, *pb = &beta_f;
  rocblas_datatype io = rocblas_datatype_f32_r, compute = rocblas_datatype_f32_r;
  if (dtype == MSHADOW_HIP_BLAS_F64) {
    io = compute = rocblas_datatype_f64_r;
    pa = &alpha;
    pb = &beta;
  } else if (dtype == MSHADOW_HIP_BLAS_F16) {
    io = rocblas_datatype_f16_r;
  }
  return FromRocBlas(
      Api().rocblas_gemm_strided_batched_ex(h, Op(transa), Op(transb), m, n, k, pa, A, io, lda,
                                            stride_a, B, io, ldb, stride_b, pb, C, io, ldc,
                                            stride_c, C, io, ldc, stride_c, batch, compute,
                                            rocblas_gemm_algo_standard, 0, 0),
      "rocblas_gemm_strided_batched_ex");
}

int mshadow_hip_blas_gemv(int dtype, int trans, int m, int n, double alpha, const void *A,
                          int lda, long long stride_a, const void *x, int incx,
                          long long stride_x, double beta, void *y, int incy,
                          long long stride_y, int batch, void *stream) {
  ABI_REQUIRE(dtype == MSHADOW_HIP_BLAS_F32 || dtype == MSHADOW_HIP_BLAS_F64,
              "gemv exists for float and double");
  ABI_REQUIRE(m >= 0 && n >= 0, "negative dimension");
  ABI_REQUIRE(BatchOk(batch, stride_a, stride_x, stride_y), "negative batch count or stride");
  ABI_REQUIRE(LeadingOk(lda, m), "lda is smaller than m");
  ABI_REQUIRE(incx != 0 && incy != 0, "zero increment");
  if (m == 0 || n == 0 || batch == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(A != nullptr && x != nullptr && y != nullptr, "null operand");
  rocblas_handle h;
  int st = HandleFor(stream, &h);
  if (st != MSHADOW_HIP_OK) return st;
  if (dtype == MSHADOW_HIP_BLAS_F32) {
    const float a = static_cast<float>(alpha), b = static_cast<float>(beta);
    return FromRocBlas(Api().rocblas_sgemv_strided_batched(
                           h, Op(trans), m, n, &a, static_cast<const float *>(A), lda, stride_a,
                           static_cast<const float *>(x), incx, stride_x, &b,
                           static_cast<float *>(y), incy, stride_y, batch),
                       "rocblas_sgemv_strided_batched");
  }
  return FromRocBlas(Api().rocblas_dgemv_strided_batched(
                         h, Op(trans), m, n, &alpha, static_cast<const double *>(A), lda,
                         stride_a, static_cast<const double *>(x), incx, stride_x, &beta,
                         static_cast<double *>(y), incy, stride_y, batch),
                     "rocblas_dgemv_strided_batched");
}

int mshadow_hip_blas_ger(int dtype, int m, int n, double alpha, const void *x, int incx,
                         long long stride_x, const void *y, int incy, long long stride_y,
                         void *A, int lda, long long stride_a, int batch, void *stream) {
  ABI_REQUIRE(dtype == MSHADOW_HIP_BLAS_F32 || dtype == MSHADOW_HIP_BLAS_F64,
              "ger exists for float and double");
  ABI_REQUIRE(m >= 0 && n >= 0, "negative dimension");
  ABI_REQUIRE(BatchOk(batch, stride_x, stride_y, stride_a), "negative batch count or stride");
  ABI_REQUIRE(LeadingOk(lda, m), "lda is smaller than m");
  ABI_REQUIRE(incx != 0 && incy != 0, "zero increment");
  if (m == 0 || n == 0 || batch == 0) return MSHADOW_HIP_OK;
  ABI_REQUIRE(A != nullptr && x != nullptr && y != nullptr, "null operand");
  ABI_REQUIRE(batch == 1 || stride_a >= static_cast<long long>(lda) * n,
              "the results of a batch overlap");
  rocblas_handle h;
  int st = HandleFor(stream, &h);
  if (st != MSHADOW_HIP_OK) return st;
  if (dtype == MSHADOW_HIP_BLAS_F32) {
    const float a = static_cast<float>(alpha);
    return FromRocBlas(Api().rocblas_sger_strided_batched(
                           h, m, n, &a, static_cast<const float *>(x), incx, stride_x,
                           static_cast<const float *>(y), incy, stride_y,
                           static_cast<float *>(A), lda, stride_a, batch),
                       "rocblas_sger_strided_batched");
  }
  return FromRocBlas(Api().rocblas_dger_strided_batched(
                         h, m, n, &alpha, static_cast<const double *>(x), incx, stride_x,
                         static_cast<const double *>(y), incy, stride_y,
                         static_cast<double *>(A), lda, stride_a, batch),
                     "rocblas_dger_strided_batched");
}

int mshadow_hip_blas_dot(int dtype, int n, const void *x, int incx, const void *y, int incy,
                         void *result, void *stream) {
  ABI_REQUIRE(dtype == MSHADOW_HIP_BLAS_F32 || dtype == MSHADOW_HIP_BLAS_F64,
              "dot exists for float and double");
  ABI_REQUIRE(n >= 0, "negative length");
  ABI_REQUIRE(result != nullptr && (n == 0 || (x != nullptr && y != nullptr)), "null operand");
  rocblas_handle h;
  int st = HandleFor(stream, &h);
  if (st != MSHADOW_HIP_OK) return st;
  /* the result stays on the device (dot_engine-inl.h:712-718); the handle is host-mode
     for every other call of this file, so the mode is put back before returning */
  st = FromRocBlas(Api().rocblas_set_pointer_mode(h, rocblas_pointer_mode_device),
                   "rocblas_set_pointer_mode");
  if (st != MSHADOW_HIP_OK) return st;
  rocblas_status rs;
  if (dtype == MSHADOW_HIP_BLAS_F32) {
    rs = Api().rocblas_sdot(h, n, static_cast<const float *>(x), incx,
                            static_cast<const float *>(y), incy, static_cast<float *>(result));
  } else {
    rs = Api().rocblas_ddot(h, n, static_cast<const double *>(x), incx,
                            static_cast<const double *>(y), incy, static_cast<double *>(result));
  }
  const rocblas_status back = Api().rocblas_set_pointer_mode(h, rocblas_pointer_mode_host);
  st = FromRocBlas(rs, "rocblas_dot");
  if (st != MSHADOW_HIP_OK) return st;
  return FromRocBlas(back, "rocblas_set_pointer_mode");
}

}  // extern "C"
