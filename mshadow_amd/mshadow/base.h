/*
 * Scalar types, type flags and the functor vocabulary (op / sv / red) of the
 * mshadow API. Names, template shapes and numeric semantics follow
 * mshadow/base.h:288-862 of the reference; see core/functors.h for the functors.
 */
#ifndef MSHADOW_BASE_H_
#define MSHADOW_BASE_H_

#include <stdint.h>
#include <cfloat>
#include <climits>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <string>

#include "./core/config.h"
#include "./half.h"
#include "./half2.h"
#include "./logging.h"

namespace mshadow {
/*! \brief buffer size for each random number generator */
const unsigned kRandBufferSize = 1000000;
/*! \brief pi */
const float kPi = 3.1415926f;
/*! \brief type that will be used for index (mshadow/base.h:288-292) */
#if MSHADOW_INT64_TENSOR_SIZE == 1
typedef int64_t index_t;
#else
typedef int32_t index_t;
#endif
typedef index_t openmp_index_t;
/*! \brief float point type that will be used in default by mshadow */
typedef float default_real_t;

/*! \brief data type flag (mshadow/base.h:306-315) */
enum TypeFlag { kFloat32 = 0, kFloat64 = 1, kFloat16 = 2, kUint8 = 3, kInt32 = 4, kInt8 = 5, kInt64 = 6 };

template <typename DType>
struct DataType;
#define MSHADOW_DECLARE_DATATYPE(T, FLAG) \
  template <>                             \
  struct DataType<T> {                    \
    static const int kFlag = FLAG;        \
    static const int kLanes = 1;          \
  };
MSHADOW_DECLARE_DATATYPE(float, kFloat32)
MSHADOW_DECLARE_DATATYPE(double, kFloat64)
MSHADOW_DECLARE_DATATYPE(half::half_t, kFloat16)
MSHADOW_DECLARE_DATATYPE(uint8_t, kUint8)
MSHADOW_DECLARE_DATATYPE(int8_t, kInt8)
MSHADOW_DECLARE_DATATYPE(int32_t, kInt32)
MSHADOW_DECLARE_DATATYPE(int64_t, kInt64)
#undef MSHADOW_DECLARE_DATATYPE
/*! \brief two binary16 lanes per element (mshadow/base.h:361-365) */
template <>
struct DataType<half::half2_t> {
  static const int kFlag = kFloat16;
  static const int kLanes = 2;
};
/*! \brief type enum value for default real type */
const int default_type_flag = DataType<default_real_t>::kFlag;

/*! \brief layout flag (mshadow/base.h:419-431) */
enum LayoutFlag { kNCHW = 0, kNHWC, kCHWN, kNCW = 1 << 3, kNWC, kCWN, kNCDHW = 1 << 5, kNDHWC, kCDHWN };
template <int layout>
struct LayoutType;
template <>
struct LayoutType<kNCHW> {
  static const index_t kNdim = 4;
};
template <>
struct LayoutType<kNHWC> {
  static const index_t kNdim = 4;
};
template <>
struct LayoutType<kNCDHW> {
  static const index_t kNdim = 5;
};
template <>
struct LayoutType<kNDHWC> {
  static const index_t kNdim = 5;
};
const int default_layout = kNCHW;
const int default_layout_5d = kNCDHW;
}  // namespace mshadow

#include "./core/functors.h"

/* ---- run-time type dispatch (mshadow/base.h:864-1100) ---- */
#define MSHADOW_SWITCH_CASE_(flag, T, DType, ...) \
  case flag: {                                    \
    typedef T DType;                              \
    { __VA_ARGS__ }                               \
  } break;
#define MSHADOW_SWITCH_END_(type) \
  default:                        \
    LOG(FATAL) << "Unknown type enum " << type;

#define MSHADOW_TYPE_SWITCH(type, DType, ...)                                      \
  switch (type) {                                                                  \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat32, float, DType, __VA_ARGS__)             \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat64, double, DType, __VA_ARGS__)            \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat16, mshadow::half::half_t, DType, __VA_ARGS__) \
    MSHADOW_SWITCH_CASE_(mshadow::kUint8, uint8_t, DType, __VA_ARGS__)             \
    MSHADOW_SWITCH_CASE_(mshadow::kInt8, int8_t, DType, __VA_ARGS__)               \
    MSHADOW_SWITCH_CASE_(mshadow::kInt32, int32_t, DType, __VA_ARGS__)             \
    MSHADOW_SWITCH_CASE_(mshadow::kInt64, int64_t, DType, __VA_ARGS__)             \
    MSHADOW_SWITCH_END_(type)                                                      \
  }
/*! \brief MSHADOW_TYPE_SWITCH without int8, with binary16 taken two lanes at a time
 *  (mshadow/base.h:919-959) */
#define MSHADOW_TYPE_SWITCH_WITH_HALF2(type, DType, ...)                            \
  switch (type) {                                                                   \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat32, float, DType, __VA_ARGS__)              \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat64, double, DType, __VA_ARGS__)             \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat16, mshadow::half::half2_t, DType, __VA_ARGS__) \
    MSHADOW_SWITCH_CASE_(mshadow::kUint8, uint8_t, DType, __VA_ARGS__)              \
    MSHADOW_SWITCH_CASE_(mshadow::kInt32, int32_t, DType, __VA_ARGS__)              \
    MSHADOW_SWITCH_CASE_(mshadow::kInt64, int64_t, DType, __VA_ARGS__)              \
    MSHADOW_SWITCH_END_(type)                                                       \
  }

#define MSHADOW_SGL_DBL_TYPE_SWITCH(type, DType, ...)                   \
  switch (type) {                                                       \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat32, float, DType, __VA_ARGS__)  \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat64, double, DType, __VA_ARGS__) \
    MSHADOW_SWITCH_END_(type)                                           \
  }
#define MSHADOW_REAL_TYPE_SWITCH(type, DType, ...)                                     \
  switch (type) {                                                                      \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat32, float, DType, __VA_ARGS__)                 \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat64, double, DType, __VA_ARGS__)                \
    MSHADOW_SWITCH_CASE_(mshadow::kFloat16, mshadow::half::half_t, DType, __VA_ARGS__) \
    case mshadow::kUint8:                                                              \
    case mshadow::kInt8:                                                               \
    case mshadow::kInt32:                                                              \
    case mshadow::kInt64:                                                              \
      LOG(FATAL) << "This operation only support floating point types not integer";    \
      break;                                                                           \
    MSHADOW_SWITCH_END_(type)                                                          \
  }
/*! \brief floating-point types only, with a second name for the type sums are kept in:
 *  float for binary16 (mshadow/base.h:1013-1055) */
#define MSHADOW_REAL_TYPE_SWITCH_EX(type, DType, DLargeType, ...)                           \
  switch (type) {                                                                           \
    case mshadow::kFloat32: {                                                               \
      typedef float DType;                                                                  \
      typedef float DLargeType;                                                             \
      { __VA_ARGS__ }                                                                       \
    } break;                                                                                \
    case mshadow::kFloat64: {                                                               \
      typedef double DType;                                                                 \
      typedef double DLargeType;                                                            \
      { __VA_ARGS__ }                                                                       \
    } break;                                                                                \
    case mshadow::kFloat16: {                                                               \
      typedef mshadow::half::half_t DType;                                                  \
      typedef float DLargeType;                                                             \
      { __VA_ARGS__ }                                                                       \
    } break;                                                                                \
    case mshadow::kUint8:                                                                   \
      LOG(FATAL) << "This operation only support floating point types not uint8";           \
      break;                                                                                \
    case mshadow::kInt8:                                                                    \
      LOG(FATAL) << "This operation only support floating point types not int8";            \
      break;                                                                                \
    case mshadow::kInt32:                                                                   \
      LOG(FATAL) << "This operation only support floating point types, not int32";          \
      break;                                                                                \
    case mshadow::kInt64:                                                                   \
      LOG(FATAL) << "This operation only support floating point types, not int64";          \
      break;                                                                                \
    default:                                                                                \
      LOG(FATAL) << "Unknown type enum " << type;                                           \
  }

#define MSHADOW_IDX_TYPE_SWITCH(type, DType, ...)                         \
  switch (type) {                                                         \
    MSHADOW_SWITCH_CASE_(mshadow::kInt32, int32_t, DType, __VA_ARGS__)    \
    MSHADOW_SWITCH_CASE_(mshadow::kInt64, int64_t, DType, __VA_ARGS__)    \
    MSHADOW_SWITCH_END_(type)                                             \
  }
#define MSHADOW_LAYOUT_SWITCH(layout, Layout, ...)    \
  switch (layout) {                                   \
    case mshadow::kNCHW: {                            \
      const int Layout = mshadow::kNCHW;              \
      { __VA_ARGS__ }                                 \
    } break;                                          \
    case mshadow::kNHWC: {                            \
      const int Layout = mshadow::kNHWC;              \
      { __VA_ARGS__ }                                 \
    } break;                                          \
    case mshadow::kNCDHW: {                           \
      const int Layout = mshadow::kNCDHW;             \
      { __VA_ARGS__ }                                 \
    } break;                                          \
    case mshadow::kNDHWC: {                           \
      const int Layout = mshadow::kNDHWC;             \
      { __VA_ARGS__ }                                 \
    } break;                                          \
    default:                                          \
      LOG(FATAL) << "Unknown layout enum " << layout; \
  }

/*! \brief get data type size from type enum */
inline size_t mshadow_sizeof(int type) {
  size_t size = 0;
  MSHADOW_TYPE_SWITCH(type, DType, size = sizeof(DType););
  return size;
}

#endif  // MSHADOW_BASE_H_
