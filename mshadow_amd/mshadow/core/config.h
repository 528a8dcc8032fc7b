/*
 * Build configuration of the gfx950 mshadow backend.
 *
 * The macro names callers may set are the reference's (mshadow/base.h:49-158,
 * :192-224): MSHADOW_ALLOC_PAD, MSHADOW_MIN_PAD_RATIO, MSHADOW_FORCE_STREAM,
 * MSHADOW_INT64_TENSOR_SIZE, MSHADOW_DEFAULT_DTYPE. There is one GPU target, so no
 * backend-selection switch changes anything here (the reference's are defined for callers
 * that test them): a translation unit built by hipcc sees device code, one built by a host
 * compiler sees the host-side API only.
 */
#ifndef MSHADOW_CORE_CONFIG_H_
#define MSHADOW_CORE_CONFIG_H_

/*! \brief pad rows of newly allocated tensors to an aligned pitch by default */
#ifndef MSHADOW_ALLOC_PAD
#define MSHADOW_ALLOC_PAD true
#endif
/*! \brief x dimension must be at least this many times the alignment unit to be padded */
#ifndef MSHADOW_MIN_PAD_RATIO
#define MSHADOW_MIN_PAD_RATIO 2
#endif
/*! \brief a NULL Stream<gpu> is a fatal error instead of meaning the default stream */
#ifndef MSHADOW_FORCE_STREAM
#define MSHADOW_FORCE_STREAM 1
#endif
#ifndef MSHADOW_INT64_TENSOR_SIZE
#define MSHADOW_INT64_TENSOR_SIZE 0
#endif

/*! \brief the GPU device of this build; kept for callers that test it */
#define MSHADOW_USE_HIP 1

/* The switches of the reference's base.h (:49-158, :226-231) that callers test with #if. This
   backend reads none of them; the values say what a caller finds here: Tensor<gpu> exists
   (MSHADOW_USE_CUDA is the reference's name for that and is 1 there by default too), matrix
   products need no external host BLAS, and there is no cuDNN, cuSOLVER, NVML or glog. */
#ifndef MSHADOW_USE_CUDA
#define MSHADOW_USE_CUDA 1
#endif
#ifndef MSHADOW_USE_CUDNN
#define MSHADOW_USE_CUDNN 0
#endif
#ifndef MSHADOW_USE_CUSOLVER
#define MSHADOW_USE_CUSOLVER 0
#endif
#ifndef MSHADOW_USE_CBLAS
#define MSHADOW_USE_CBLAS 0
#endif
#ifndef MSHADOW_USE_MKL
#define MSHADOW_USE_MKL 0
#endif
#ifndef MSHADOW_STAND_ALONE
#define MSHADOW_STAND_ALONE 0
#endif
#ifndef MSHADOW_OLD_CUDA
#define MSHADOW_OLD_CUDA 0
#endif
#ifndef MSHADOW_IN_CXX11
#define MSHADOW_IN_CXX11 1
#endif
#ifndef MSHADOW_USE_SSE
#define MSHADOW_USE_SSE 0
#endif
#ifndef MSHADOW_USE_F16C
#if defined(__F16C__) && !defined(__HIP_DEVICE_COMPILE__)
#define MSHADOW_USE_F16C 1  /* half.h converts with the host's F16C instructions */
#else
#define MSHADOW_USE_F16C 0
#endif
#endif
#ifndef MSHADOW_USE_NVML
#define MSHADOW_USE_NVML 0
#endif
#ifndef MSHADOW_USE_GLOG
#define MSHADOW_USE_GLOG 0
#endif

#ifdef MSHADOW_XINLINE
#error "MSHADOW_XINLINE must not be defined"
#endif
#define MSHADOW_FORCE_INLINE inline __attribute__((always_inline))
#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define MSHADOW_XINLINE MSHADOW_FORCE_INLINE __device__ __host__
#else
#define MSHADOW_XINLINE MSHADOW_FORCE_INLINE
#endif
#define MSHADOW_CINLINE MSHADOW_FORCE_INLINE
#define MSHADOW_CONSTEXPR constexpr
#define MSHADOW_ALIGNED(x) __attribute__((aligned(x)))
#define MSHADOW_THROW_EXCEPTION noexcept(false)
#define MSHADOW_NO_EXCEPTION noexcept(true)

#ifndef MSHADOW_DEFAULT_DTYPE
#define MSHADOW_DEFAULT_DTYPE = ::mshadow::default_real_t
#endif

#endif  // MSHADOW_CORE_CONFIG_H_
