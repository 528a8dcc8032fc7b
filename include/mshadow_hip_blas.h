/*
 * C ABI of the dense linear-algebra entry points of the gfx950 mshadow backend: what
 * BLASEngine<gpu, DType> of the reference binds to cuBLAS (mshadow/dot_engine-inl.h:501-838).
 *
 * These are plain library GEMM / GEMV / GER / DOT calls: the library forwards them to
 * rocBLAS, which it opens on the first call (a process that never multiplies matrices never
 * loads it; one whose system has no rocBLAS gets MSHADOW_HIP_ERR_UNSUPPORTED with the loader's
 * message). Everything is column-major with leading dimensions in elements, exactly as the
 * reference passes it; a batch is `batch` problems `stride_*` elements apart (batch 1 and
 * strides 0 for a single problem), which replaces the pointer-array workspace of the
 * reference's batched calls. alpha and beta travel as double and are narrowed to the
 * computation type: float for MSHADOW_HIP_BLAS_F32 and _F16 (binary16 storage, float
 * accumulation, as the reference's cublasSgemmEx call), double for _F64.
 * All pointers are device pointers; the call is queued on `stream` and returns at once.
 * Return codes and error text as in mshadow_hip.h.
 */
#ifndef MSHADOW_HIP_BLAS_H_
#define MSHADOW_HIP_BLAS_H_

#include "mshadow_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define MSHADOW_HIP_BLAS_F32 0
#define MSHADOW_HIP_BLAS_F64 1
#define MSHADOW_HIP_BLAS_F16 2 /* gemm only, as in the reference (dot_engine-inl.h:570-603) */

/* C = alpha * op(A) * op(B) + beta * C, C is m x n, op(A) m x k, op(B) k x n:
   BLASEngine<gpu, DType>::gemm and ::batched_gemm, dot_engine-inl.h:511-568, :615-668,
   :732-785 (cublasSgemm / Dgemm / SgemmEx and their strided-batched forms). */
int mshadow_hip_blas_gemm(int dtype, int transa, int transb, int m, int n, int k, double alpha,
                          const void *A, int lda, long long stride_a, const void *B, int ldb,
                          long long stride_b, double beta, void *C, int ldc, long long stride_c,
                          int batch, void *stream);
/* y = alpha * op(A) * x + beta * y, A is m x n: ::gemv and ::batched_gemv,
   dot_engine-inl.h:670-688, :787-805 (cublasSgemv / Dgemv). */
int mshadow_hip_blas_gemv(int dtype, int trans, int m, int n, double alpha, const void *A,
                          int lda, long long stride_a, const void *x, int incx,
                          long long stride_x, double beta, void *y, int incy,
                          long long stride_y, int batch, void *stream);
/* A += alpha * x * y^T, A is m x n: ::ger and ::batched_ger, dot_engine-inl.h:690-705,
   :807-822 (cublasSger / Dger). */
int mshadow_hip_blas_ger(int dtype, int m, int n, double alpha, const void *x, int incx,
                         long long stride_x, const void *y, int incy, long long stride_y,
                         void *A, int lda, long long stride_a, int batch, void *stream);
/* *result = sum_i x[i] * y[i], result in device memory: ::dot, dot_engine-inl.h:707-719,
   :824-836 (cublasSdot / Ddot in device pointer mode). */
int mshadow_hip_blas_dot(int dtype, int n, const void *x, int incx, const void *y, int incy,
                         void *result, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MSHADOW_HIP_BLAS_H_ */
