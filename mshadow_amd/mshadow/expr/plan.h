/*
 * Plan<Exp, DType>: the by-value, device-copyable evaluator of an expression tree.
 *
 * MakePlan(tree) flattens the reference-linked tree into nested Plan objects holding
 * raw pointers, pitches and scalars; `plan.Eval(y, x)` yields the element of the 2-D
 * view at row y, column x. This is the contract of mshadow/expr_engine-inl.h:39-232
 * in the reference (Plan / MakePlan are extension points: callers specialise Plan for
 * their own nodes and only need Eval).
 *
 * Added for gfx950: plans made only of tensors, scalars and elementwise maps also
 * evaluate N adjacent columns at once (EvalPack<N>) from one 128-bit global load per
 * tensor leaf. A plan advertises that with `kPackable`; PackReady() checks at run
 * time that every leaf pointer and pitch is aligned for N-wide access. EvalPack's second
 * template argument asks the leaves for non-temporal (streaming) accesses. Chainer plans
 * that read their source at the column they are asked for (row remappings, windows over
 * rows) forward packs too; they clear *flat in PackReady because they need the real row
 * number. Plans without these members (caller-defined ones) simply take the scalar path.
 */
#ifndef MSHADOW_EXPR_PLAN_H_
#define MSHADOW_EXPR_PLAN_H_

#include <stdint.h>

#include "../core/tensor_types.h"

namespace mshadow {
namespace expr {

/*! \brief N adjacent elements of a row, aligned so that one memory instruction moves them */
template <typename DType, int N>
struct MSHADOW_ALIGNED(sizeof(DType) * N) Pack {
  DType v[N];
};

namespace plan_detail {
/*! \brief raw 128/64/32-bit vector used to move a Pack with one memory instruction */
template <int BYTES>
struct RawVec {
#if defined(__clang__)
  typedef uint32_t type __attribute__((ext_vector_type(BYTES / 4)));
#else
  struct type { uint32_t w[BYTES / 4]; };  // host compilers never issue the streaming forms
#endif
};
template <>
struct RawVec<4> {
  typedef uint32_t type;
};
template <>
struct RawVec<2> {
  typedef uint16_t type;
};
template <>
struct RawVec<1> {
  typedef uint8_t type;
};
/*! \brief load / store one Pack. STREAM marks the access non-temporal: the data passes
 *  through once and should not displace other lines in the caches (device code only). */
/* On the device a pack is moved as one access wherever it lies: the address needs the
   element's alignment only (16-byte global accesses need no 16-byte alignment on gfx950; where
   the address happens to be aligned the instruction is the same one). */
template <typename DType, int N, bool STREAM>
MSHADOW_XINLINE Pack<DType, N> LoadPack(const DType *p) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename RawVec<sizeof(DType) * N>::type Raw;
  typedef Raw Loose __attribute__((aligned(1)));
  Raw raw;
  if (STREAM) {
    raw = __builtin_nontemporal_load(reinterpret_cast<const Loose *>(p));
  } else {
    raw = *reinterpret_cast<const Loose *>(p);
  }
  Pack<DType, N> out;
  __builtin_memcpy(&out, &raw, sizeof(out));
  return out;
#else
  return *reinterpret_cast<const Pack<DType, N> *>(p);
#endif
}
template <typename DType, int N, bool STREAM>
MSHADOW_XINLINE void StorePackTo(DType *p, const Pack<DType, N> &v) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename RawVec<sizeof(DType) * N>::type Raw;
  typedef Raw Loose __attribute__((aligned(1)));
  Raw raw;
  __builtin_memcpy(&raw, &v, sizeof(raw));
  if (STREAM) {
    __builtin_nontemporal_store(raw, reinterpret_cast<Loose *>(p));
  } else {
    *reinterpret_cast<Loose *>(p) = raw;
  }
#else
  *reinterpret_cast<Pack<DType, N> *>(p) = v;
#endif
}
}  // namespace plan_detail

/*! \brief base of the chainer nodes: a node that knows its own output shape */
template <typename SubType, typename SrcExp, int dim, typename DType>
struct MakeTensorExp : public Exp<MakeTensorExp<SubType, SrcExp, dim, DType>, DType, type::kChainer> {
  /*! \brief shape of the output */
  Shape<dim> shape_;
  inline const SubType &real_self(void) const { return *static_cast<const SubType *>(this); }
};

template <typename ExpType, typename DType>
class Plan {
 public:
  /*! \brief value at row y, column x of the flattened 2-D view */
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const;
};

/* ---- leaves ---- */
template <typename Device, int dim, typename DType>
class Plan<Tensor<Device, dim, DType>, DType> {
 public:
  static const bool kPackable = true;
  static const bool kRaggedRows = true;
  explicit Plan(const Tensor<Device, dim, DType> &t) : dptr_(t.dptr_), stride_(t.stride_) {}
  /* offsets in 64 bits whatever index_t is: a tensor whose dimensions each fit index_t may
     still hold 2^31 elements or more (65536 x 32768 floats are 8 GiB of a 288 GB device) */
  MSHADOW_XINLINE DType &REval(index_t y, index_t x) { return dptr_[At(y, x)]; }
  MSHADOW_XINLINE const DType &Eval(index_t y, index_t x) const { return dptr_[At(y, x)]; }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    return plan_detail::LoadPack<DType, N, STREAM>(dptr_ + At(y, x));
  }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE void StorePack(index_t y, index_t x, const Pack<DType, N> &p) {
    plan_detail::StorePackTo<DType, N, STREAM>(dptr_ + At(y, x), p);
  }
  /*! \brief host check: pointer and pitch allow n-wide access; *flat stays true only
   *  while rows are dense (pitch == cols) so that the 2-D view can be walked linearly */
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    if (stride_ != cols) *flat = false;
    return true;  // a pack is fetched wherever it lies
  }

 private:
  MSHADOW_XINLINE int64_t At(index_t y, index_t x) const {
    return static_cast<int64_t>(y) * stride_ + x;
  }
  DType *dptr_;
  index_t stride_;
};

template <typename Device, typename DType>
class Plan<Tensor<Device, 1, DType>, DType> {
 public:
  static const bool kPackable = true;
  static const bool kRaggedRows = true;
  explicit Plan(const Tensor<Device, 1, DType> &t) : dptr_(t.dptr_) {}
  MSHADOW_XINLINE DType &REval(index_t y, index_t x) { return dptr_[x]; }
  MSHADOW_XINLINE const DType &Eval(index_t y, index_t x) const { return dptr_[x]; }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    return plan_detail::LoadPack<DType, N, STREAM>(dptr_ + x);
  }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE void StorePack(index_t y, index_t x, const Pack<DType, N> &p) {
    plan_detail::StorePackTo<DType, N, STREAM>(dptr_ + x, p);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const { return true; }

 private:
  DType *dptr_;
};

template <typename DType>
class Plan<ScalarExp<DType>, DType> {
 public:
  static const bool kPackable = true;
  static const bool kRaggedRows = true;
  explicit Plan(DType scalar) : scalar_(scalar) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const { return scalar_; }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    Pack<DType, N> p;
#pragma unroll
    for (int i = 0; i < N; ++i) p.v[i] = scalar_;
    return p;
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const { return true; }

 private:
  DType scalar_;
};

/*! \brief rows of one plane of the destination when somewhere in the plan a window runs
 *  over neighbouring planes (channel pooling), 0 otherwise: the launcher then hands each
 *  thread packs of adjacent planes, so that a window's fetches are mostly repeats of the
 *  thread's own. Plans say so with a PlaneRows() member; any plan may go without. */
template <typename P>
inline auto PlaneRowsOf(const P &plan, int) -> decltype(plan.PlaneRows()) {
  return plan.PlaneRows();
}
template <typename P>
inline index_t PlaneRowsOf(const P &, long) {
  return 0;
}

/* ---- interior nodes ---- */
template <typename DstDType, typename SrcDType, typename EType, int etype>
class Plan<TypecastExp<DstDType, SrcDType, EType, etype>, DstDType> {
 public:
  explicit Plan(const Plan<EType, SrcDType> &src) : src_(src) {}
  MSHADOW_XINLINE DstDType Eval(index_t y, index_t x) const {
    return DstDType(src_.Eval(y, x));  // NOLINT(*)
  }

 private:
  Plan<EType, SrcDType> src_;
};

namespace plan_detail {
/*! \brief P::kPackable if the plan type declares it, false otherwise */
template <typename P>
struct Packable {
  template <typename Q>
  static char Test(int (*)[Q::kPackable ? 1 : -1]);
  template <typename Q>
  static long Test(...);  // NOLINT(*)
  static const bool value = sizeof(Test<P>(0)) == sizeof(char);
};
/*! \brief P::kRaggedRows if the plan type declares it, false otherwise: the plan is made of
 *  tensors, scalars and elementwise functions only, so it evaluates a pack at any column of
 *  any row (rows need not be whole packs, nor start at multiples of 16 bytes) */
template <typename P>
struct RaggedRows {
  template <typename Q>
  static char Test(int (*)[Q::kRaggedRows ? 1 : -1]);
  template <typename Q>
  static long Test(...);  // NOLINT(*)
  static const bool value = sizeof(Test<P>(0)) == sizeof(char);
};
/*! \brief P::kPlaneWindow if the plan type declares it, false otherwise: somewhere in the
 *  plan a window runs over neighbouring planes, and the plan has EvalPackRun */
template <typename P>
struct PlaneWindow {
  template <typename Q>
  static char Test(int (*)[Q::kPlaneWindow ? 1 : -1]);
  template <typename Q>
  static long Test(...);  // NOLINT(*)
  static const bool value = sizeof(Test<P>(0)) == sizeof(char);
};
template <bool kWindow>
struct RunOf {
  template <int N, bool STREAM, int K, typename P, typename DType>
  MSHADOW_XINLINE static void Eval(const P &plan, index_t y0, index_t dy, index_t x,
                                   Pack<DType, N> *out) {
#pragma unroll
    for (int u = 0; u < K; ++u) out[u] = plan.template EvalPack<N, STREAM>(y0 + u * dy, x);
  }
};
template <>
struct RunOf<true> {
  template <int N, bool STREAM, int K, typename P, typename DType>
  MSHADOW_XINLINE static void Eval(const P &plan, index_t y0, index_t dy, index_t x,
                                   Pack<DType, N> *out) {
    plan.template EvalPackRun<N, STREAM, K>(y0, dy, x, out);
  }
};
}  // namespace plan_detail

/*! \brief out[u] = plan.EvalPack(y0 + u * dy, x) for u < K: the same place of K planes that
 *  are dy rows apart. A plan with a window over planes shares the fetches of overlapping
 *  windows (its EvalPackRun); every other plan evaluates the K packs one by one. */
template <int N, bool STREAM, int K, typename P, typename DType>
MSHADOW_XINLINE void EvalPackRun(const P &plan, index_t y0, index_t dy, index_t x,
                                 Pack<DType, N> *out) {
  plan_detail::RunOf<plan_detail::PlaneWindow<P>::value>::template Eval<N, STREAM, K>(plan, y0, dy,
                                                                                      x, out);
}

template <typename OP, typename TA, typename TB, typename TC, int etype, typename DType>
class Plan<TernaryMapExp<OP, TA, TB, TC, DType, etype>, DType> {
 public:
  static const bool kPackable = plan_detail::Packable<Plan<TA, DType> >::value &&
                                plan_detail::Packable<Plan<TB, DType> >::value &&
                                plan_detail::Packable<Plan<TC, DType> >::value;
  static const bool kRaggedRows = plan_detail::RaggedRows<Plan<TA, DType> >::value &&
                                  plan_detail::RaggedRows<Plan<TB, DType> >::value &&
                                  plan_detail::RaggedRows<Plan<TC, DType> >::value;
  explicit Plan(const Plan<TA, DType> &item1, const Plan<TB, DType> &item2,
                const Plan<TC, DType> &item3)
      : item1_(item1), item2_(item2), item3_(item3) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    return OP::Map(item1_.Eval(y, x), item2_.Eval(y, x), item3_.Eval(y, x));
  }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    const Pack<DType, N> a = item1_.template EvalPack<N, STREAM>(y, x);
    const Pack<DType, N> b = item2_.template EvalPack<N, STREAM>(y, x);
    const Pack<DType, N> c = item3_.template EvalPack<N, STREAM>(y, x);
    Pack<DType, N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = OP::Map(a.v[i], b.v[i], c.v[i]);
    return r;
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    return item1_.PackReady(n, cols, flat) && item2_.PackReady(n, cols, flat) &&
           item3_.PackReady(n, cols, flat);
  }

 private:
  Plan<TA, DType> item1_;
  Plan<TB, DType> item2_;
  Plan<TC, DType> item3_;
};

template <typename OP, typename TA, typename TB, int etype, typename DType>
class Plan<BinaryMapExp<OP, TA, TB, DType, etype>, DType> {
 public:
  static const bool kPackable = plan_detail::Packable<Plan<TA, DType> >::value &&
                                plan_detail::Packable<Plan<TB, DType> >::value;
  static const bool kRaggedRows = plan_detail::RaggedRows<Plan<TA, DType> >::value &&
                                  plan_detail::RaggedRows<Plan<TB, DType> >::value;
  explicit Plan(const Plan<TA, DType> &lhs, const Plan<TB, DType> &rhs) : lhs_(lhs), rhs_(rhs) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const {
    return OP::Map(lhs_.Eval(y, x), rhs_.Eval(y, x));
  }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    const Pack<DType, N> a = lhs_.template EvalPack<N, STREAM>(y, x);
    const Pack<DType, N> b = rhs_.template EvalPack<N, STREAM>(y, x);
    Pack<DType, N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = OP::Map(a.v[i], b.v[i]);
    return r;
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    return lhs_.PackReady(n, cols, flat) && rhs_.PackReady(n, cols, flat);
  }
  inline index_t PlaneRows() const {
    const index_t l = PlaneRowsOf(lhs_, 0);
    return l != 0 ? l : PlaneRowsOf(rhs_, 0);
  }
  static const bool kPlaneWindow = plan_detail::PlaneWindow<Plan<TA, DType> >::value ||
                                   plan_detail::PlaneWindow<Plan<TB, DType> >::value;
  template <int N, bool STREAM, int K>
  MSHADOW_XINLINE void EvalPackRun(index_t y0, index_t dy, index_t x, Pack<DType, N> *out) const {
    Pack<DType, N> a[K], b[K];
    expr::EvalPackRun<N, STREAM, K>(lhs_, y0, dy, x, a);
    expr::EvalPackRun<N, STREAM, K>(rhs_, y0, dy, x, b);
#pragma unroll
    for (int u = 0; u < K; ++u) {
#pragma unroll
      for (int i = 0; i < N; ++i) out[u].v[i] = OP::Map(a[u].v[i], b[u].v[i]);
    }
  }

 private:
  Plan<TA, DType> lhs_;
  Plan<TB, DType> rhs_;
};

template <typename OP, typename TA, int etype, typename DType>
class Plan<UnaryMapExp<OP, TA, DType, etype>, DType> {
 public:
  static const bool kPackable = plan_detail::Packable<Plan<TA, DType> >::value;
  static const bool kRaggedRows = plan_detail::RaggedRows<Plan<TA, DType> >::value;
  explicit Plan(const Plan<TA, DType> &src) : src_(src) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const { return OP::Map(src_.Eval(y, x)); }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    const Pack<DType, N> a = src_.template EvalPack<N, STREAM>(y, x);
    Pack<DType, N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = OP::Map(a.v[i]);
    return r;
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    return src_.PackReady(n, cols, flat);
  }
  inline index_t PlaneRows() const { return PlaneRowsOf(src_, 0); }
  static const bool kPlaneWindow = plan_detail::PlaneWindow<Plan<TA, DType> >::value;
  template <int N, bool STREAM, int K>
  MSHADOW_XINLINE void EvalPackRun(index_t y0, index_t dy, index_t x, Pack<DType, N> *out) const {
    expr::EvalPackRun<N, STREAM, K>(src_, y0, dy, x, out);
#pragma unroll
    for (int u = 0; u < K; ++u) {
#pragma unroll
      for (int i = 0; i < N; ++i) out[u].v[i] = OP::Map(out[u].v[i]);
    }
  }

 private:
  Plan<TA, DType> src_;
};

/*! \brief a chainer node evaluates through the plan of its concrete type */
template <typename SubType, typename SrcExp, int dim, typename DType>
struct Plan<MakeTensorExp<SubType, SrcExp, dim, DType>, DType> {
 public:
  /*! \brief a chainer that keeps the column of its source (a remapping of rows, a window
   *  over rows) can evaluate packs; its concrete plan says so */
  static const bool kPackable = plan_detail::Packable<Plan<SubType, DType> >::value;
  Plan(const Plan<SubType, DType> &src) : src_(src) {}  // NOLINT(*)
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const { return src_.Eval(y, x); }
  template <int N, bool STREAM = false>
  MSHADOW_XINLINE Pack<DType, N> EvalPack(index_t y, index_t x) const {
    return src_.template EvalPack<N, STREAM>(y, x);
  }
  inline bool PackReady(int n, index_t cols, bool *flat) const {
    return src_.PackReady(n, cols, flat);
  }
  inline index_t PlaneRows() const { return PlaneRowsOf(src_, 0); }
  static const bool kPlaneWindow = plan_detail::PlaneWindow<Plan<SubType, DType> >::value;
  template <int N, bool STREAM, int K>
  MSHADOW_XINLINE void EvalPackRun(index_t y0, index_t dy, index_t x, Pack<DType, N> *out) const {
    expr::EvalPackRun<N, STREAM, K>(src_, y0, dy, x, out);
  }

 private:
  Plan<SubType, DType> src_;
};

template <typename EType, typename DType>
class Plan<TransposeExp<EType, DType>, DType> {
 public:
  explicit Plan(const Plan<EType, DType> &src) : src_(src) {}
  MSHADOW_XINLINE DType Eval(index_t y, index_t x) const { return src_.Eval(x, y); }

 private:
  Plan<EType, DType> src_;
};

/* ---- MakePlan: tree -> plan (mshadow/expr_engine-inl.h:175-232) ---- */
template <typename OP, typename TA, typename TB, typename DType, int etype>
inline Plan<BinaryMapExp<OP, TA, TB, DType, etype>, DType> MakePlan(
    const BinaryMapExp<OP, TA, TB, DType, etype> &e);
template <typename OP, typename TA, typename TB, typename TC, typename DType, int etype>
inline Plan<TernaryMapExp<OP, TA, TB, TC, DType, etype>, DType> MakePlan(
    const TernaryMapExp<OP, TA, TB, TC, DType, etype> &e);

template <typename DType>
inline Plan<ScalarExp<DType>, DType> MakePlan(const ScalarExp<DType> &e) {
  return Plan<ScalarExp<DType>, DType>(e.scalar_);
}
template <typename DstDType, typename SrcDType, typename EType, int etype>
inline Plan<TypecastExp<DstDType, SrcDType, EType, etype>, DstDType> MakePlan(
    const TypecastExp<DstDType, SrcDType, EType, etype> &e) {
  return Plan<TypecastExp<DstDType, SrcDType, EType, etype>, DstDType>(MakePlan(e.exp));
}
template <typename T, typename DType>
inline Plan<T, DType> MakePlan(const RValueExp<T, DType> &e) {
  return Plan<T, DType>(e.self());
}
template <typename T, typename DType>
inline Plan<TransposeExp<T, DType>, DType> MakePlan(const TransposeExp<T, DType> &e) {
  return Plan<TransposeExp<T, DType>, DType>(MakePlan(e.exp));
}
template <typename T, typename SrcExp, int dim, typename DType>
inline Plan<T, DType> MakePlan(const MakeTensorExp<T, SrcExp, dim, DType> &e) {
  return Plan<T, DType>(e.real_self());
}
template <typename OP, typename TA, typename DType, int etype>
inline Plan<UnaryMapExp<OP, TA, DType, etype>, DType> MakePlan(
    const UnaryMapExp<OP, TA, DType, etype> &e) {
  return Plan<UnaryMapExp<OP, TA, DType, etype>, DType>(MakePlan(e.src_));
}
template <typename OP, typename TA, typename TB, typename DType, int etype>
inline Plan<BinaryMapExp<OP, TA, TB, DType, etype>, DType> MakePlan(
    const BinaryMapExp<OP, TA, TB, DType, etype> &e) {
  return Plan<BinaryMapExp<OP, TA, TB, DType, etype>, DType>(MakePlan(e.lhs_), MakePlan(e.rhs_));
}
template <typename OP, typename TA, typename TB, typename TC, typename DType, int etype>
inline Plan<TernaryMapExp<OP, TA, TB, TC, DType, etype>, DType> MakePlan(
    const TernaryMapExp<OP, TA, TB, TC, DType, etype> &e) {
  return Plan<TernaryMapExp<OP, TA, TB, TC, DType, etype>, DType>(
      MakePlan(e.item1_), MakePlan(e.item2_), MakePlan(e.item3_));
}

}  // namespace expr
}  // namespace mshadow
#endif  // MSHADOW_EXPR_PLAN_H_
