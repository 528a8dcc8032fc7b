/*
 * Build configuration of the gfx950 mshadow backend.
 *
 * The macro names callers may set are the reference's (mshadow/base.h:49-158,
 * :192-224): MSHADOW_ALLOC_PAD, MSHADOW_MIN_PAD_RATIO, MSHADOW_FORCE_STREAM,
 * MSHADOW_INT64_TENSOR_SIZE, MSHADOW_DEFAULT_DTYPE. There is one GPU target, so no
 * backend-selection switches exist: a translation unit built by hipcc sees device
 * code, one built by a host compiler sees the host-side API only.
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
