/*
 * Random<Device, DType>: a seeded source of random tensors.
 *
 * Interface of mshadow/random.h:33-568 of the reference. On the CPU the engine is
 * std::mt19937 and every sampler is the standard library's distribution of that name driven
 * element by element in row-major order, so a given seed yields the values the reference
 * yields when both are built against the same standard library. On the GPU the reference
 * asks cuRAND; here the values come from the library's counter-based Philox generator
 * (mshadow_hip_random_*): reproducible for a seed, independent of launch shape, and - like
 * any pair of different generators - not equal to cuRAND's or to the CPU's. The object keeps
 * (seed, blocks consumed); Seed() rewinds.
 */
#ifndef MSHADOW_RANDOM_H_
#define MSHADOW_RANDOM_H_

#include <algorithm>
#include <cstdlib>
#include <random>
#include <type_traits>

#include "./base.h"
#include "./tensor.h"
#include "./tensor_container.h"

namespace mshadow {

template <typename Device, typename DType MSHADOW_DEFAULT_DTYPE>
class Random {};

template <typename DType>
class Random<cpu, DType> {
 public:
  explicit Random(int seed) {
    this->Seed(seed);
    buffer_.Resize(Shape1(kRandBufferSize));
  }
  inline void Seed(int seed) {
    rnd_engine_.seed(seed);
    rseed_ = static_cast<unsigned>(seed);
  }
  inline unsigned GetSeed() const { return rseed_; }
  inline void set_stream(Stream<cpu> *) {}
  inline unsigned GetRandInt() { return rnd_engine_(); }
  inline void GetRandInt(const Tensor<cpu, 1, unsigned> &dst) {
    for (index_t i = 0; i < dst.size(0); ++i) dst.dptr_[i] = rnd_engine_();
  }
  /*! \brief one draw of `sampler` per element, rows in order (the pitch gap is skipped) */
  template <int dim, class Sampler>
  inline void SampleDistribution(Tensor<cpu, dim, DType> *dst, Sampler sampler) {
    Tensor<cpu, 2, DType> mat = dst->FlatTo2D();
    for (index_t y = 0; y < mat.size(0); ++y) {
      DType *row = mat[y].dptr_;
      for (index_t x = 0; x < mat.size(1); ++x) row[x] = sampler();
    }
  }
  /*! \brief uniform on [a, b) for floating types, on [a, b] for integer types */
  template <int dim, typename PType>
  inline void SampleUniform(Tensor<cpu, dim, DType> *dst, PType a = 0.0f, PType b = 1.0f) {
    typedef typename std::conditional<std::is_floating_point<DType>::value, DType, double>::type FType;
    typedef typename std::conditional<std::is_integral<DType>::value,
                                      std::uniform_int_distribution<DType>,
                                      std::uniform_real_distribution<FType> >::type Dist;
    Dist dist(a, b);
    SampleDistribution(dst, [&]() { return dist(rnd_engine_); });
  }
  template <int dim, typename PType>
  inline void SampleGaussian(Tensor<cpu, dim, DType> *dst, PType mu = 0.0f, PType sigma = 1.0f) {
    if (sigma <= 0) {
      *dst = mu;
      return;
    }
    std::normal_distribution<typename Real<DType>::type> dist(mu, sigma);
    SampleDistribution(dst, [&]() { return dist(rnd_engine_); });
  }
  template <int dim, typename PType>
  inline void SampleGamma(Tensor<cpu, dim, DType> *dst, PType alpha, PType beta) {
    std::gamma_distribution<typename Real<DType>::type> dist(alpha, beta);
    SampleDistribution(dst, [&]() { return dist(rnd_engine_); });
  }
  template <int dim, typename PType>
  inline void SampleExponential(Tensor<cpu, dim, DType> *dst, PType lambda) {
    std::exponential_distribution<typename Real<DType>::type> dist(lambda);
    SampleDistribution(dst, [&]() { return dist(rnd_engine_); });
  }
  template <int dim, typename PType>
  inline void SamplePoisson(Tensor<cpu, dim, DType> *dst, PType lambda) {
    std::poisson_distribution<typename Count<DType>::type> dist(lambda);
    SampleDistribution(dst, [&]() { return static_cast<DType>(dist(rnd_engine_)); });
  }
  template <int dim, typename PType1, typename PType2>
  inline void SampleNegativeBinomial(Tensor<cpu, dim, DType> *dst, PType1 k, PType2 p) {
    std::negative_binomial_distribution<typename Count<DType>::type> dist(k, p);
    SampleDistribution(dst, [&]() { return static_cast<DType>(dist(rnd_engine_)); });
  }
  /*! \brief Poisson whose rate is Gamma(1 / alpha, mu * alpha) distributed; plain Poisson(mu)
   *  when alpha is 0 */
  template <int dim, typename PType>
  inline void SampleGeneralizedNegativeBinomial(Tensor<cpu, dim, DType> *dst, PType mu,
                                                PType alpha) {
    if (alpha == PType(0)) {
      SamplePoisson(dst, mu);
      return;
    }
    std::gamma_distribution<> rate(PType(1) / alpha, mu * alpha);
    SampleDistribution(dst, [&]() {
      std::poisson_distribution<typename Count<DType>::type> dist(rate(rnd_engine_));
      return static_cast<DType>(dist(rnd_engine_));
    });
  }
  /*! \brief standard normal values of the given shape, valid until the next call */
  template <int dim>
  inline expr::ReshapeExp<Tensor<cpu, 1, DType>, DType, dim, 1> gaussian(Shape<dim> shape) {
    buffer_.Resize(Shape1(shape.Size()));
    this->SampleGaussian(&buffer_, 0.0f, 1.0f);
    return expr::reshape(buffer_, shape);
  }
  /*! \brief uniform [0, 1) values of the given shape, valid until the next call */
  template <int dim>
  inline expr::ReshapeExp<Tensor<cpu, 1, DType>, DType, dim, 1> uniform(Shape<dim> shape) {
    buffer_.Resize(Shape1(shape.Size()));
    this->SampleUniform(&buffer_, 0.0f, 1.0f);
    return expr::reshape(buffer_, shape);
  }
  std::mt19937 &GetRndEngine() { return rnd_engine_; }

 private:
  /* samplers of real-valued distributions work in DType when it is a floating type, else in
     double; counting distributions in DType when it is an integer type, else in int */
  template <typename T>
  struct Real {
    typedef typename std::conditional<std::is_floating_point<T>::value, T, double>::type type;
  };
  template <typename T>
  struct Count {
    typedef typename std::conditional<std::is_integral<T>::value, T, int>::type type;
  };
  std::mt19937 rnd_engine_;
  unsigned rseed_;
  TensorContainer<cpu, 1, DType> buffer_;
};

template <typename DType>
class Random<gpu, DType> {
 public:
  explicit Random(int seed) : stream_(NULL) {
    this->Seed(seed);
    buffer_.Resize(Shape1(kRandBufferSize));
  }
  /*! \brief the stream the sampling kernels are queued on */
  inline void set_stream(Stream<gpu> *stream) {
    stream_ = stream;
    buffer_.set_stream(stream);
  }
  /*! \brief start the sequence of this seed from its beginning */
  inline void Seed(int seed) {
    seed_ = static_cast<uint64_t>(static_cast<int64_t>(seed));
    counter_ = 0;
  }
  inline void GetRandInt(const Tensor<gpu, 1, unsigned> &dst) {
    MSHADOW_HIP_CALL(mshadow_hip_random_u32(dst.dptr_, dst.size(0), seed_, 0, counter_, Raw()));
    Advance((static_cast<size_t>(dst.size(0)) + 3) / 4);
  }
  template <int dim>
  inline void SampleUniform(Tensor<gpu, dim, DType> *dst, DType a = 0.0f, DType b = 1.0f) {
    const Shape<2> s = dst->shape_.FlatTo2D();
    Advance(Draw(0, dst->dptr_, dst->stride_, s[0], s[1], a, b));
  }
  template <int dim>
  inline void SampleGaussian(Tensor<gpu, dim, DType> *dst, DType mu = 0.0f, DType sigma = 1.0f) {
    const Shape<2> s = dst->shape_.FlatTo2D();
    Advance(Draw(1, dst->dptr_, dst->stride_, s[0], s[1], mu, sigma));
  }
  /*! \brief normal values of the given shape, valid until the next call */
  template <int dim>
  inline expr::ReshapeExp<Tensor<gpu, 1, DType>, DType, dim, 1> gaussian(Shape<dim> shape,
                                                                        DType mu = 0.0f,
                                                                        DType sigma = 1.0f) {
    buffer_.Resize(Shape1(shape.Size()));
    this->SampleGaussian(&buffer_, mu, sigma);
    return expr::reshape(buffer_, shape);
  }
  /*! \brief uniform (0, 1) values of the given shape, valid until the next call */
  template <int dim>
  inline expr::ReshapeExp<Tensor<gpu, 1, DType>, DType, dim, 1> uniform(Shape<dim> shape) {
    buffer_.Resize(Shape1(shape.Size()));
    this->SampleUniform(&buffer_, 0.0f, 1.0f);
    return expr::reshape(buffer_, shape);
  }

 private:
  inline void *Raw() { return Stream<gpu>::GetStream(stream_); }
  inline void Advance(size_t blocks) { counter_ += blocks; }
  /*! \brief kind 0 uniform (p0, p1), 1 normal (mean p0, deviation p1); returns the generator
   *  blocks the call consumed: four floats or two doubles come out of one */
  inline size_t Draw(int kind, float *dst, index_t stride, index_t rows, index_t cols, float p0,
                     float p1) {
    if (kind == 0) {
      MSHADOW_HIP_CALL(mshadow_hip_random_uniform_f32(dst, stride, rows, cols, seed_, 0, counter_,
                                                      p0, p1, Raw()));
    } else {
      MSHADOW_HIP_CALL(mshadow_hip_random_normal_f32(dst, stride, rows, cols, seed_, 0, counter_,
                                                     p0, p1, Raw()));
    }
    return (static_cast<size_t>(rows) * cols + 3) / 4;
  }
  inline size_t Draw(int kind, double *dst, index_t stride, index_t rows, index_t cols, double p0,
                     double p1) {
    if (kind == 0) {
      MSHADOW_HIP_CALL(mshadow_hip_random_uniform_f64(dst, stride, rows, cols, seed_, 0, counter_,
                                                      p0, p1, Raw()));
    } else {
      MSHADOW_HIP_CALL(mshadow_hip_random_normal_f64(dst, stride, rows, cols, seed_, 0, counter_,
                                                     p0, p1, Raw()));
    }
    return (static_cast<size_t>(rows) * cols + 1) / 2;
  }
  /*! \brief any other element type: the class itself instantiates (an operator templated over
   *  DType may hold a Random<gpu, DType> it never samples from), sampling does not compile,
   *  as with the float* / double* overloads of mshadow/random.h:486-514 */
  template <typename T>
  inline size_t Draw(int, T *, index_t, index_t, index_t, T, T) {
    static_assert(std::is_same<T, float>::value || std::is_same<T, double>::value,
                  "Random<gpu, DType> samples float and double, the types the reference's "
                  "generator library serves (mshadow/random.h:486-514)");
    return 0;
  }
  Stream<gpu> *stream_;
  uint64_t seed_;
  uint64_t counter_;
  TensorContainer<gpu, 1, DType> buffer_;
};

}  // namespace mshadow
#endif  // MSHADOW_RANDOM_H_
