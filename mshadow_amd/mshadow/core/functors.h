/*
 * Elementwise operators (op::), assignment savers (sv::) and reducers (red::).
 *
 * These are template arguments of the expression engine; user code supplies more of
 * the same shape (a struct with a static, MSHADOW_XINLINE Map / Save / Reduce). The
 * numeric behaviour restates mshadow/base.h:483-862 of the reference:
 *   - sv::X::Save(a, b) is `a X= b` on the element type;
 *   - red::maximum / minimum use operator< exactly like std::max / std::min
 *     (first argument wins ties, so -0 / +0 and NaN follow that rule, not fmax);
 *   - their initial values are the most negative / positive *finite* value;
 *   - PartialGrad of maximum / minimum is an equality test on the stored values.
 * The reference declares the reducer arguments volatile (a CUDA warp-synchronous
 * idiom); here they are plain references so that accumulators stay in registers.
 * Reducers written by callers in either style work with both devices.
 */
#ifndef MSHADOW_CORE_FUNCTORS_H_
#define MSHADOW_CORE_FUNCTORS_H_

namespace mshadow {
/*! \brief namespace for operators */
namespace op {
/*! \brief mul operator */
struct mul {
  template <typename DType>
  MSHADOW_XINLINE static DType Map(DType a, DType b) { return a * b; }
};
/*! \brief plus operator */
struct plus {
  template <typename DType>
  MSHADOW_XINLINE static DType Map(DType a, DType b) { return a + b; }
};
/*! \brief minus operator */
struct minus {
  template <typename DType>
  MSHADOW_XINLINE static DType Map(DType a, DType b) { return a - b; }
};
/*! \brief divide operator */
struct div {
  template <typename DType>
  MSHADOW_XINLINE static DType Map(DType a, DType b) { return a / b; }
};
/*! \brief get rhs */
struct right {
  template <typename DType>
  MSHADOW_XINLINE static DType Map(DType a, DType b) { return b; }
};
/*! \brief identity function */
struct identity {
  template <typename DType>
  MSHADOW_XINLINE static DType Map(DType a) { return a; }
};
}  // namespace op

/*! \brief namespace for savers */
namespace sv {
#define MSHADOW_DEFINE_SAVER(NAME, STMT, OPTYPE, ALPHA, BETA)               \
  struct NAME {                                                             \
    template <typename DType>                                               \
    MSHADOW_XINLINE static void Save(DType &a, DType b) { STMT; } /* NOLINT(*) */ \
    inline static default_real_t AlphaBLAS(void) { return ALPHA; }          \
    inline static default_real_t BetaBLAS(void) { return BETA; }            \
    typedef op::OPTYPE OPType;                                              \
  };
/*! \brief save to saver: = */
MSHADOW_DEFINE_SAVER(saveto, a = b, right, 1.0f, 0.0f)
/*! \brief save to saver: += */
MSHADOW_DEFINE_SAVER(plusto, a += b, plus, 1.0f, 1.0f)
/*! \brief minus to saver: -= */
MSHADOW_DEFINE_SAVER(minusto, a -= b, minus, -1.0f, 1.0f)
#undef MSHADOW_DEFINE_SAVER
/*! \brief multiply to saver: *= */
struct multo {
  template <typename DType>
  MSHADOW_XINLINE static void Save(DType &a, DType b) { a *= b; }  // NOLINT(*)
  typedef op::mul OPType;
};
/*! \brief divide to saver: /= */
struct divto {
  template <typename DType>
  MSHADOW_XINLINE static void Save(DType &a, DType b) { a /= b; }  // NOLINT(*)
  typedef op::div OPType;
};
}  // namespace sv

/*! \brief namespace for potential reducer operations */
namespace red {
namespace limits {
/*! \brief minimum finite value of a type */
template <typename DType>
MSHADOW_XINLINE DType MinValue(void);
/*! \brief maximum finite value of a type */
template <typename DType>
MSHADOW_XINLINE DType MaxValue(void);
#define MSHADOW_DEFINE_LIMITS(T, LO, HI)             \
  template <>                                        \
  MSHADOW_XINLINE T MinValue<T>(void) { return LO; } \
  template <>                                        \
  MSHADOW_XINLINE T MaxValue<T>(void) { return HI; }
MSHADOW_DEFINE_LIMITS(float, -FLT_MAX, FLT_MAX)
MSHADOW_DEFINE_LIMITS(double, -DBL_MAX, DBL_MAX)
MSHADOW_DEFINE_LIMITS(uint8_t, 0, UCHAR_MAX)
MSHADOW_DEFINE_LIMITS(int8_t, SCHAR_MIN, SCHAR_MAX)
MSHADOW_DEFINE_LIMITS(int32_t, INT_MIN, INT_MAX)
MSHADOW_DEFINE_LIMITS(int64_t, LLONG_MIN, LLONG_MAX)
#undef MSHADOW_DEFINE_LIMITS
template <>
MSHADOW_XINLINE half::half_t MinValue<half::half_t>(void) { return MSHADOW_HALF_MIN; }
template <>
MSHADOW_XINLINE half::half_t MaxValue<half::half_t>(void) { return MSHADOW_HALF_MAX; }
}  // namespace limits

/*! \brief sum reducer */
struct sum {
  /*! \brief do reduction into dst */
  template <typename DType>
  MSHADOW_XINLINE static void Reduce(DType &dst, DType src) {  // NOLINT(*)
    dst += src;
  }
  /*! \brief Kahan-compensated reduction, residual carried by the caller */
  template <typename DType>
  MSHADOW_XINLINE static void Reduce(DType &dst, DType src,  // NOLINT(*)
                                     DType &residual) {               // NOLINT(*)
    DType y = src - residual;
    DType t = dst + y;
    residual = (t - dst) - y;
    dst = t;
  }
  /*! \brief combine the results of two reducers */
  template <typename DType>
  MSHADOW_XINLINE static void Merge(DType &dst_val, DType &src_val) {  // NOLINT(*)
    Reduce(dst_val, src_val);
  }
  template <typename DType>
  MSHADOW_XINLINE static void Merge(DType &dst_val, DType &dst_residual,  // NOLINT(*)
                                    DType &src_val, DType &src_residual) {  // NOLINT(*)
    DType t1 = dst_val + src_val;
    DType e = t1 - dst_val;
    DType t2 = ((src_val - e) + (dst_val - (t1 - e))) + dst_residual + src_residual;
    dst_val = t1 + t2;
    dst_residual = t2 - (dst_val - t1);
  }
  template <typename DType>
  MSHADOW_XINLINE static void Finalize(DType &dst) {}  // NOLINT(*)
  template <typename DType>
  MSHADOW_XINLINE static void Finalize(DType &dst, DType &residual) {}  // NOLINT(*)
  /*! \brief d(result)/d(source element) */
  template <typename DType>
  MSHADOW_XINLINE static DType PartialGrad(DType redres, DType redsrc) { return 1; }
  /*! \brief value a reduction starts from */
  template <typename DType>
  MSHADOW_XINLINE static void SetInitValue(DType &initv) { initv = 0; }  // NOLINT(*)
  template <typename DType>
  MSHADOW_XINLINE static void SetInitValue(DType &initv, DType &residual) {  // NOLINT(*)
    SetInitValue(initv);
    residual = 0;
  }
};

#define MSHADOW_DEFINE_EXTREMUM(NAME, PICK, INIT)                                              \
  struct NAME {                                                                                \
    template <typename DType>                                                                  \
    MSHADOW_XINLINE static void Reduce(DType &dst, DType src) { /* NOLINT */ \
      const DType d = dst, s = src;                                                            \
      dst = (PICK) ? s : d;                                                                    \
    }                                                                                          \
    template <typename DType>                                                                  \
    MSHADOW_XINLINE static void Reduce(DType &dst, DType src,   /* NOLINT */ \
                                       DType &none) {                    /* NOLINT */ \
      Reduce(dst, src);                                                                        \
    }                                                                                          \
    template <typename DType>                                                                  \
    MSHADOW_XINLINE static void Merge(DType &dst_val, DType &src_val) { /* NOLINT */ \
      Reduce(dst_val, src_val);                                                                \
    }                                                                                          \
    template <typename DType>                                                                  \
    MSHADOW_XINLINE static void Merge(DType &dst_val, DType &dst_residual, /* NOLINT */ \
                                      DType &src_val, DType &src_residual) { /* NOLINT */ \
      Reduce(dst_val, src_val);                                                                \
    }                                                                                          \
    template <typename DType>                                                                  \
    MSHADOW_XINLINE static void Finalize(DType &dst) {} /* NOLINT */                  \
    template <typename DType>                                                                  \
    MSHADOW_XINLINE static void Finalize(DType &dst, DType &residual) {} /* NOLINT */ \
    template <typename DType>                                                                  \
    MSHADOW_XINLINE static DType PartialGrad(DType redres, DType redsrc) {                     \
      return redres == redsrc ? 1 : 0;                                                         \
    }                                                                                          \
    template <typename DType>                                                                  \
    MSHADOW_XINLINE static void SetInitValue(DType &initv) { /* NOLINT */                      \
      initv = limits::INIT<DType>();                                                           \
    }                                                                                          \
    template <typename DType>                                                                  \
    MSHADOW_XINLINE static void SetInitValue(DType &initv, DType &none) { /* NOLINT */         \
      SetInitValue(initv);                                                                     \
    }                                                                                          \
  };
/*! \brief maximum reducer: dst = std::max(dst, src) = (dst < src) ? src : dst */
MSHADOW_DEFINE_EXTREMUM(maximum, d < s, MinValue)
/*! \brief minimum reducer: dst = std::min(dst, src) = (src < dst) ? src : dst */
MSHADOW_DEFINE_EXTREMUM(minimum, s < d, MaxValue)
#undef MSHADOW_DEFINE_EXTREMUM
}  // namespace red
}  // namespace mshadow
#endif  // MSHADOW_CORE_FUNCTORS_H_
