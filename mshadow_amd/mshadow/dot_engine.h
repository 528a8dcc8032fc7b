/*
 * Matrix products: `dst <saver>= scale * dot(lhs[.T()], rhs[.T()])`, VectorDot, BatchGEMM.
 *
 * Contract: mshadow/dot_engine-inl.h and mshadow/expr_engine-inl.h:464-479 of the reference.
 * The expression engine hands a DotExp of two tensors to DotEngine, which turns the
 * row-major product into one column-major BLAS call with the operands exchanged
 * (dot_engine-inl.h:844-933), and BLASEngine<Device, DType> is the BLAS of that device:
 *   cpu  the routines of this file - plain loops in DType, no external BLAS (the
 *        reference needs CBLAS or MKL here, and without them only knows three GEMM forms);
 *   gpu  the dense linear-algebra entry points of the C ABI (mshadow_hip_blas.h), which
 *        forward to rocBLAS on the tensor's stream.
 * Rounding: a BLAS is free to add in any order, so results agree with another BLAS to a
 * few ulp per term, not bit for bit.
 *
 * One deliberate difference: `dst = dot(x.T(), y)` of two vectors stores the outer product.
 * The reference sends exactly the storing form to BLAS ger (:922-925), which adds to what
 * dst held before; here the adding savers (+=, -=) use ger and the storing one uses gemm.
 */
#ifndef MSHADOW_DOT_ENGINE_H_
#define MSHADOW_DOT_ENGINE_H_

#include <mshadow_hip_blas.h>

#include "./tensor.h"

namespace mshadow {

/*! \brief dst[i] = src + i * stride: the pointer-array view the reference's batched cuBLAS
 *  calls need (dot_engine-inl.h:19-44); the batched routines here take strides instead, so
 *  only the host form exists */
template <typename DType>
inline void GetBatchedView(DType **dst, DType *src, int num, int stride, Stream<cpu> *stream) {
  for (int i = 0; i < num; ++i) dst[i] = src + static_cast<size_t>(i) * stride;
}

namespace expr {

/*! \brief column-major BLAS subset on the host, in DType arithmetic */
namespace cpu_blas {
template <typename DType>
inline void Gemm(bool transa, bool transb, int m, int n, int k, DType alpha, const DType *A,
                 int lda, const DType *B, int ldb, DType beta, DType *C, int ldc) {
  for (int j = 0; j < n; ++j) {
    DType *cj = C + static_cast<size_t>(j) * ldc;
    if (beta == DType(0)) {  // BLAS: C is not read when beta is zero
      for (int i = 0; i < m; ++i) cj[i] = DType(0);
    } else if (!(beta == DType(1))) {
      for (int i = 0; i < m; ++i) cj[i] = cj[i] * beta;
    }
    if (!transa) {
      for (int p = 0; p < k; ++p) {
        const DType b = alpha * (transb ? B[j + static_cast<size_t>(p) * ldb]
                                        : B[p + static_cast<size_t>(j) * ldb]);
        const DType *ap = A + static_cast<size_t>(p) * lda;
        for (int i = 0; i < m; ++i) cj[i] += b * ap[i];
      }
    } else {
      for (int i = 0; i < m; ++i) {
        const DType *ai = A + static_cast<size_t>(i) * lda;
        DType acc = DType(0);
        if (!transb) {
          const DType *bj = B + static_cast<size_t>(j) * ldb;
          for (int p = 0; p < k; ++p) acc += ai[p] * bj[p];
        } else {
          for (int p = 0; p < k; ++p) acc += ai[p] * B[j + static_cast<size_t>(p) * ldb];
        }
        cj[i] += alpha * acc;
      }
    }
  }
}
template <typename DType>
inline void Gemv(bool trans, int m, int n, DType alpha, const DType *A, int lda, const DType *X,
                 int incX, DType beta, DType *Y, int incY) {
  const int ylen = trans ? n : m;
  for (int i = 0; i < ylen; ++i) {
    DType &y = Y[static_cast<size_t>(i) * incY];
    y = (beta == DType(0)) ? DType(0) : DType(y * beta);
  }
  for (int j = 0; j < n; ++j) {
    const DType *aj = A + static_cast<size_t>(j) * lda;
    if (!trans) {
      const DType x = alpha * X[static_cast<size_t>(j) * incX];
      for (int i = 0; i < m; ++i) Y[static_cast<size_t>(i) * incY] += x * aj[i];
    } else {
      DType acc = DType(0);
      for (int i = 0; i < m; ++i) acc += aj[i] * X[static_cast<size_t>(i) * incX];
      Y[static_cast<size_t>(j) * incY] += alpha * acc;
    }
  }
}
template <typename DType>
inline void Ger(int m, int n, DType alpha, const DType *X, int incX, const DType *Y, int incY,
                DType *A, int lda) {
  for (int j = 0; j < n; ++j) {
    const DType y = alpha * Y[static_cast<size_t>(j) * incY];
    DType *aj = A + static_cast<size_t>(j) * lda;
    for (int i = 0; i < m; ++i) aj[i] += X[static_cast<size_t>(i) * incX] * y;
  }
}
}  // namespace cpu_blas

template <typename Device, typename DType MSHADOW_DEFAULT_DTYPE>
struct BLASEngine;

/*! \brief BLAS on the host; argument meaning of every routine as in dot_engine-inl.h:59-114 */
template <typename DType>
struct BLASEngine<cpu, DType> {
  inline static bool GetT(bool t) { return t; }
  inline static void SetStream(Stream<cpu> *stream) {}
  inline static void gemm(Stream<cpu> *stream, bool transa, bool transb, int m, int n, int k,
                          DType alpha, const DType *A, int lda, const DType *B, int ldb,
                          DType beta, DType *C, int ldc) {
    cpu_blas::Gemm(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc);
  }
  inline static void batched_gemm(Stream<cpu> *stream, bool transa, bool transb, int m, int n,
                                  int k, DType alpha, const DType *A, int lda, const DType *B,
                                  int ldb, DType beta, DType *C, int ldc, int batch_count,
                                  DType **workspace) {
    for (int i = 0; i < batch_count; ++i) {
      gemm(stream, transa, transb, m, n, k, alpha, A + static_cast<size_t>(i) * m * k, lda,
           B + static_cast<size_t>(i) * k * n, ldb, beta, C + static_cast<size_t>(i) * m * n,
           ldc);
    }
  }
  inline static void gemv(Stream<cpu> *stream, bool trans, int m, int n, DType alpha,
                          const DType *A, int lda, const DType *X, int incX, DType beta,
                          DType *Y, int incY) {
    cpu_blas::Gemv(trans, m, n, alpha, A, lda, X, incX, beta, Y, incY);
  }
  inline static void batched_gemv(Stream<cpu> *stream, bool trans, int m, int n, DType alpha,
                                  const DType *A, int lda, const DType *X, int incX, DType beta,
                                  DType *Y, int incY, int batch_count) {
    for (int i = 0; i < batch_count; ++i) {
      gemv(stream, trans, m, n, alpha, A + static_cast<size_t>(i) * m * n, lda,
           X + static_cast<size_t>(i) * (trans ? m : n) * incX, incX, beta,
           Y + static_cast<size_t>(i) * (trans ? n : m) * incY, incY);
    }
  }
  inline static void ger(Stream<cpu> *stream, int m, int n, DType alpha, const DType *X,
                         int incX, const DType *Y, int incY, DType *A, int lda) {
    cpu_blas::Ger(m, n, alpha, X, incX, Y, incY, A, lda);
  }
  inline static void batched_ger(Stream<cpu> *stream, int m, int n, DType alpha, const DType *X,
                                 int incX, const DType *Y, int incY, DType *A, int lda,
                                 int batch_count) {
    for (int i = 0; i < batch_count; ++i) {
      ger(stream, m, n, alpha, X + static_cast<size_t>(i) * m * incX, incX,
          Y + static_cast<size_t>(i) * n * incY, incY, A + static_cast<size_t>(i) * lda * n, lda);
    }
  }
  inline static void dot(Stream<cpu> *stream, int n, const DType *X, int incX, const DType *Y,
                         int incY, DType *ret) {
    DType acc = DType(0);
    for (int i = 0; i < n; ++i) {
      acc += X[static_cast<size_t>(i) * incX] * Y[static_cast<size_t>(i) * incY];
    }
    *ret = acc;
  }
};

namespace gpu_blas {
/*! \brief element type code of the C ABI, -1 where the device has no BLAS for the type */
template <typename DType>
struct Code {
  static const int kCode = -1;
};
template <>
struct Code<float> {
  static const int kCode = MSHADOW_HIP_BLAS_F32;
};
template <>
struct Code<double> {
  static const int kCode = MSHADOW_HIP_BLAS_F64;
};
template <>
struct Code<half::half_t> {
  static const int kCode = MSHADOW_HIP_BLAS_F16;
};
}  // namespace gpu_blas

/*! \brief BLAS on the device: float and double throughout, half_t for gemm (binary16
 *  storage, float accumulation), like dot_engine-inl.h:501-838 */
template <typename DType>
struct BLASEngine<gpu, DType> {
  static const int kCode = gpu_blas::Code<DType>::kCode;
  inline static bool GetT(bool t) { return t; }
  /*! \brief every call below passes its stream itself; kept because callers use it */
  inline static void SetStream(Stream<gpu> *stream) {}
  inline static void CheckType(bool level3_only) {
    if (kCode < 0 || (!level3_only && kCode == MSHADOW_HIP_BLAS_F16)) {
      LOG(FATAL) << "Not implmented!";
    }
  }
  inline static void gemm(Stream<gpu> *stream, bool transa, bool transb, int m, int n, int k,
                          DType alpha, const DType *A, int lda, const DType *B, int ldb,
                          DType beta, DType *C, int ldc) {
    batched_gemm(stream, transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, 1, NULL);
  }
  inline static void batched_gemm(Stream<gpu> *stream, bool transa, bool transb, int m, int n,
                                  int k, DType alpha, const DType *A, int lda, const DType *B,
                                  int ldb, DType beta, DType *C, int ldc, int batch_count,
                                  DType **workspace) {
    CheckType(true);
    MSHADOW_HIP_CALL(mshadow_hip_blas_gemm(
        kCode, transa, transb, m, n, k, static_cast<double>(alpha), A, lda,
        static_cast<long long>(m) * k, B, ldb, static_cast<long long>(k) * n,
        static_cast<double>(beta), C, ldc, static_cast<long long>(m) * n, batch_count,
        Stream<gpu>::GetStream(stream)));
  }
  inline static void gemv(Stream<gpu> *stream, bool trans, int m, int n, DType alpha,
                          const DType *A, int lda, const DType *X, int incX, DType beta,
                          DType *Y, int incY) {
    batched_gemv(stream, trans, m, n, alpha, A, lda, X, incX, beta, Y, incY, 1);
  }
  inline static void batched_gemv(Stream<gpu> *stream, bool trans, int m, int n, DType alpha,
                                  const DType *A, int lda, const DType *X, int incX, DType beta,
                                  DType *Y, int incY, int batch_count) {
    CheckType(false);
    MSHADOW_HIP_CALL(mshadow_hip_blas_gemv(
        kCode, trans, m, n, static_cast<double>(alpha), A, lda, static_cast<long long>(m) * n,
        X, incX, static_cast<long long>(trans ? m : n) * incX, static_cast<double>(beta), Y,
        incY, static_cast<long long>(trans ? n : m) * incY, batch_count,
        Stream<gpu>::GetStream(stream)));
  }
  inline static void ger(Stream<gpu> *stream, int m, int n, DType alpha, const DType *X,
                         int incX, const DType *Y, int incY, DType *A, int lda) {
    batched_ger(stream, m, n, alpha, X, incX, Y, incY, A, lda, 1);
  }
  inline static void batched_ger(Stream<gpu> *stream, int m, int n, DType alpha, const DType *X,
                                 int incX, const DType *Y, int incY, DType *A, int lda,
                                 int batch_count) {
    CheckType(false);
    MSHADOW_HIP_CALL(mshadow_hip_blas_ger(
        kCode, m, n, static_cast<double>(alpha), X, incX, static_cast<long long>(m) * incX, Y,
        incY, static_cast<long long>(n) * incY, A, lda, static_cast<long long>(lda) * n,
        batch_count, Stream<gpu>::GetStream(stream)));
  }
  /*! \brief ret is device memory; the call is queued like every other */
  inline static void dot(Stream<gpu> *stream, int n, const DType *X, int incX, const DType *Y,
                         int incY, DType *ret) {
    CheckType(false);
    MSHADOW_HIP_CALL(mshadow_hip_blas_dot(kCode, n, X, incX, Y, incY, ret,
                                          Stream<gpu>::GetStream(stream)));
  }
};

template <typename SV, typename Device, int ddim, int ldim, int rdim, bool ltrans, bool rtrans,
          typename DType>
struct DotEngine {
  inline static void Eval(Tensor<Device, ddim, DType> *p_dst,
                          const Tensor<Device, ldim, DType> &lhs,
                          const Tensor<Device, rdim, DType> &rhs, DType scale);
};

/*! \brief The reference built without an external BLAS (MSHADOW_STAND_ALONE, which is what this
 *  device is compared with) evaluates dst = dot(A, B), dot(A, B.T()) and dot(A.T(), B) on the
 *  host through implicit_dot (dot_engine-inl.h:853-863): four partial sums per element, folded
 *  (s0 + s2) + (s1 + s3). The host device takes the same route for those three forms, so its
 *  products agree with that build bit for bit; every other form (a scale, a saver other than
 *  `=`, both operands transposed) runs the plain loops of BLASEngine<cpu>. */
template <typename SV, typename xpu, bool transpose_left, bool transpose_right, typename DType>
struct HostProduct {
  inline static bool Run(Tensor<xpu, 2, DType> *, const Tensor<xpu, 2, DType> &,
                         const Tensor<xpu, 2, DType> &, DType) {
    return false;
  }
};
template <bool transpose_left, bool transpose_right, typename DType>
struct HostProduct<sv::saveto, cpu, transpose_left, transpose_right, DType> {
  inline static bool Run(Tensor<cpu, 2, DType> *dst, const Tensor<cpu, 2, DType> &lhs,
                         const Tensor<cpu, 2, DType> &rhs, DType scale) {
    if (!(scale == DType(1.0f)) || (transpose_left && transpose_right)) return false;
    if (transpose_left) {
      *dst = expr::implicit_dot(lhs.T(), rhs);
    } else if (transpose_right) {
      *dst = expr::implicit_dot(lhs, rhs.T());
    } else {
      *dst = expr::implicit_dot(lhs, rhs);
    }
    return true;
  }
};

inline Shape<2> GetShape(const Shape<2> &shape, bool transpose) {
  return transpose ? Shape2(shape[1], shape[0]) : shape;
}

/*! \brief matrix x matrix. Row-major dst = L R is column-major dst^T = R^T L^T, so the
 *  right operand goes first */
template <typename SV, typename xpu, bool transpose_left, bool transpose_right, typename DType>
struct DotEngine<SV, xpu, 2, 2, 2, transpose_left, transpose_right, DType> {
  inline static void Eval(Tensor<xpu, 2, DType> *p_dst, const Tensor<xpu, 2, DType> &lhs,
                          const Tensor<xpu, 2, DType> &rhs, DType scale) {
    Tensor<xpu, 2, DType> &dst = *p_dst;
    if (HostProduct<SV, xpu, transpose_left, transpose_right, DType>::Run(p_dst, lhs, rhs, scale)) return;
    BLASEngine<xpu, DType>::SetStream(dst.stream_);
    Shape<2> sleft = GetShape(lhs.shape_, transpose_left);
    Shape<2> sright = GetShape(rhs.shape_, transpose_right);
    CHECK(dst.size(0) == sleft[0] && dst.size(1) == sright[1] && sleft[1] == sright[0])
        << "dot-gemm: matrix shape mismatch";
    BLASEngine<xpu, DType>::gemm(dst.stream_, transpose_right, transpose_left,
                                 transpose_right ? rhs.size(0) : rhs.size(1),
                                 transpose_left ? lhs.size(1) : lhs.size(0),
                                 transpose_right ? rhs.size(1) : rhs.size(0),
                                 DType(scale * SV::AlphaBLAS()), rhs.dptr_, rhs.stride_,
                                 lhs.dptr_, lhs.stride_, DType(SV::BetaBLAS()), dst.dptr_,
                                 dst.stride_);
  }
};
/*! \brief vector x matrix */
template <typename SV, typename xpu, bool transpose_right, typename DType>
struct DotEngine<SV, xpu, 1, 1, 2, false, transpose_right, DType> {
  inline static void Eval(Tensor<xpu, 1, DType> *p_dst, const Tensor<xpu, 1, DType> &lhs,
                          const Tensor<xpu, 2, DType> &rhs, DType scale) {
    Tensor<xpu, 1, DType> &dst = *p_dst;
    BLASEngine<xpu, DType>::SetStream(dst.stream_);
    Shape<2> sright = GetShape(rhs.shape_, transpose_right);
    CHECK(dst.size(0) == sright[1] && lhs.size(0) == sright[0])
        << "dot-gemv: matrix shape mismatch"
        << "dst: " << dst.shape_ << "\n"
        << "lhs: " << lhs.shape_ << "\n"
        << "rhs: " << sright << "\n";
    BLASEngine<xpu, DType>::gemv(dst.stream_, transpose_right, rhs.size(1), rhs.size(0),
                                 DType(scale * SV::AlphaBLAS()), rhs.dptr_, rhs.stride_,
                                 lhs.dptr_, 1, DType(SV::BetaBLAS()), dst.dptr_, 1);
  }
};
/*! \brief outer product of two vectors */
template <typename SV, typename xpu, typename DType>
struct DotEngine<SV, xpu, 2, 1, 1, true, false, DType> {
  inline static void Eval(Tensor<xpu, 2, DType> *p_dst, const Tensor<xpu, 1, DType> &lhs,
                          const Tensor<xpu, 1, DType> &rhs, DType scale) {
    Tensor<xpu, 2, DType> &dst = *p_dst;
    BLASEngine<xpu, DType>::SetStream(dst.stream_);
    CHECK(dst.size(0) == lhs.size(0) && dst.size(1) == rhs.size(0))
        << "dot-ger: matrix shape mismatch"
        << "dst: " << dst.shape_ << "\n"
        << "lhs: " << lhs.shape_ << "\n"
        << "rhs: " << rhs.shape_;
    if (SV::BetaBLAS() == 1.0f) {  // ger adds to dst
      BLASEngine<xpu, DType>::ger(dst.stream_, rhs.size(0), lhs.size(0),
                                  DType(scale * SV::AlphaBLAS()), rhs.dptr_, 1, lhs.dptr_, 1,
                                  dst.dptr_, dst.stride_);
    } else {
      DotEngine<SV, xpu, 2, 2, 2, true, false, DType>::Eval(p_dst, lhs.FlatTo2D(),
                                                            rhs.FlatTo2D(), scale);
    }
  }
};
/*! \brief batch of matrix products, the engine behind batch_dot (expression.h:244-249 of
 *  the reference declares the expression) */
template <typename SV, typename xpu, bool transpose_left, bool transpose_right, typename DType>
struct DotEngine<SV, xpu, 3, 3, 3, transpose_left, transpose_right, DType> {
  inline static void Eval(Tensor<xpu, 3, DType> *p_dst, const Tensor<xpu, 3, DType> &lhs,
                          const Tensor<xpu, 3, DType> &rhs, DType scale) {
    BatchGEMM<transpose_left, transpose_right>(*p_dst, lhs, rhs, DType(scale * SV::AlphaBLAS()),
                                               DType(SV::BetaBLAS()),
                                               Tensor<xpu, 1, DType *>(NULL, Shape1(0)));
  }
};

template <typename SV, typename Device, int dim, int ldim, int rdim, bool ltrans, bool rtrans,
          typename DType>
struct ExpComplexEngine<SV, Tensor<Device, dim, DType>,
                        DotExp<Tensor<Device, ldim, DType>, Tensor<Device, rdim, DType>, ltrans,
                               rtrans, DType>,
                        DType> {
  inline static void Eval(Tensor<Device, dim, DType> *dst,
                          const DotExp<Tensor<Device, ldim, DType>, Tensor<Device, rdim, DType>,
                                       ltrans, rtrans, DType> &exp) {
    DotEngine<SV, Device, dim, ldim, rdim, ltrans, rtrans, DType>::Eval(dst, exp.lhs_, exp.rhs_,
                                                                        exp.scale_);
  }
};

}  // namespace expr

template <typename Device, typename DType>
inline void VectorDot(Tensor<Device, 1, DType> dst, const Tensor<Device, 1, DType> &lhs,
                      const Tensor<Device, 1, DType> &rhs) {
  CHECK_EQ(lhs.size(0), rhs.size(0)) << "VectorDot: Shape mismatch";
  CHECK_EQ(dst.size(0), 1U) << "VectorDot: expect dst to be scalar";
  expr::BLASEngine<Device, DType>::SetStream(lhs.stream_);
  expr::BLASEngine<Device, DType>::dot(lhs.stream_, lhs.size(0), lhs.dptr_, 1, rhs.dptr_, 1,
                                       dst.dptr_);
}

/*! \brief the batches are found by stride, so `workspace` (room for 3 * batch pointers in
 *  the reference, tensor.h:1037-1053) is accepted and not used: an empty one will do */
template <bool transpose_left, bool transpose_right, typename Device, typename DType>
inline void BatchGEMM(Tensor<Device, 3, DType> dst, const Tensor<Device, 3, DType> &lhs,
                      const Tensor<Device, 3, DType> &rhs, DType alpha, DType beta,
                      Tensor<Device, 1, DType *> workspace) {
  index_t batch_size = dst.shape_[0];
  expr::BLASEngine<Device, DType>::SetStream(dst.stream_);
  Shape<3> sleft =
      transpose_left ? Shape3(lhs.shape_[0], lhs.shape_[2], lhs.shape_[1]) : lhs.shape_;
  Shape<3> sright =
      transpose_right ? Shape3(rhs.shape_[0], rhs.shape_[2], rhs.shape_[1]) : rhs.shape_;
  CHECK_EQ(dst.CheckContiguous(), true);
  CHECK_EQ(lhs.CheckContiguous(), true);
  CHECK_EQ(rhs.CheckContiguous(), true);
  CHECK(sleft[0] == batch_size && sright[0] == batch_size)
      << "BatchGEMM: batchsize must be equal."
      << "dst: " << dst.shape_ << "\n"
      << "lhs: " << sleft << "\n"
      << "rhs: " << sright << "\n";
  CHECK(dst.size(1) == sleft[1] && dst.size(2) == sright[2] && sleft[2] == sright[1])
      << "BatchGEMM: matrix shape mismatch"
      << "dst: " << dst.shape_ << "\n"
      << "lhs: " << sleft << "\n"
      << "rhs: " << sright << "\n";
  expr::BLASEngine<Device, DType>::batched_gemm(
      dst.stream_, transpose_right, transpose_left,
      transpose_right ? rhs.size(1) : rhs.size(2), transpose_left ? lhs.size(2) : lhs.size(1),
      transpose_right ? rhs.size(2) : rhs.size(1), alpha, rhs.dptr_, rhs.stride_, lhs.dptr_,
      lhs.stride_, beta, dst.dptr_, dst.stride_, batch_size, workspace.dptr_);
}

}  // namespace mshadow
#endif  // MSHADOW_DOT_ENGINE_H_
