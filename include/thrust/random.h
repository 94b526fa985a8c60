// thrust::random: the engines and distributions that device code draws from -- the usual way to
// make test data in place: a functor seeds an engine, discards up to its element's index and draws
// (thrust/random.h; thrust/random/linear_congruential_engine.h and detail/mod.h: x <- (a x + c) mod m;
// detail/linear_congruential_engine_discard.h: skipping ahead by modular exponentiation;
// detail/uniform_real_distribution.inl:60-80, uniform_int_distribution.inl:66-86,
// normal_distribution_base.h:80-130, the portable form that compilers other than nvcc take;
// testing/random.cu).  Everything is __host__ __device__ and gives the same numbers on both sides.
// Provided: linear_congruential_engine, minstd_rand0, minstd_rand, default_random_engine,
// uniform_real_distribution, uniform_int_distribution, normal_distribution.
#pragma once
#include <iostream>  // as the reference's header does: its users print what they draw
#include <cmath>
#include <cstdint>
#include <limits>

#include <thrust/detail/config.h>
#include <thrust/pair.h>

namespace thrust {
namespace random {
namespace detail {
// (a x + c) mod m without overflow; m == 0 means the natural modulus of the type
template <typename T, T a, T c, T m, bool Narrow = (sizeof(T) <= 4)>
struct affine_mod {
  __host__ __device__ static T apply(T x) {  // up to 32 bits: 64-bit arithmetic holds the product
    return (T)(((unsigned long long)a * x + c) % m);
  }
};
template <typename T, T a, T c, T m>
struct affine_mod<T, a, c, m, false> {
  __host__ __device__ static T apply(T x) {  // Schrage's decomposition, m = a q + r
    const T q = m / a, r = m % a;
    if (a == 1) {
      x %= m;
    } else {
      const T t1 = a * (x % q), t2 = r * (x / q);
      x = t1 >= t2 ? t1 - t2 : m - t2 + t1;
    }
    if (c != 0) {
      const T d = m - x;
      x = d > c ? x + c : c - d;
    }
    return x;
  }
};
template <typename T, T a, T c, T m>
__host__ __device__ inline T next_state(T x) {
  return m == 0 ? (T)(a * x + c) : affine_mod<T, a, c, (m == 0 ? 1 : m)>::apply(x);
}
}  // namespace detail

template <typename UIntType, UIntType a, UIntType c, UIntType m>
class linear_congruential_engine {
 public:
  typedef UIntType result_type;
  static const result_type multiplier = a;
  static const result_type increment = c;
  static const result_type modulus = m;
  static const result_type min = c == 0u ? 1u : 0u;
  static const result_type max = m - 1u;
  static const result_type default_seed = 1u;

  __host__ __device__ explicit linear_congruential_engine(result_type s = default_seed) { seed(s); }
  __host__ __device__ void seed(result_type s = default_seed) {
    const result_type sm = m == 0 ? s : (result_type)(s % (m == 0 ? 1 : m));
    const result_type cm = m == 0 ? c : (result_type)(c % (m == 0 ? 1 : m));
    x_ = (cm == 0 && sm == 0) ? (result_type)1 : sm;
  }
  __host__ __device__ result_type operator()() {
    x_ = detail::next_state<UIntType, a, c, m>(x_);
    return x_;
  }
  // z draws at once: for c == 0 and 32-bit state x <- a^z x mod m by repeated squaring
  __host__ __device__ void discard(unsigned long long z) {
    if (c == 0 && m != 0 && sizeof(UIntType) <= 4) {
      unsigned long long base = a, power = 1;
      while (z > 0) {
        if (z & 1) power = (power * base) % m;
        z >>= 1;
        base = (base * base) % m;
      }
      x_ = (result_type)((power * x_) % m);
    } else {
      for (; z > 0; --z) x_ = detail::next_state<UIntType, a, c, m>(x_);
    }
  }
  __host__ __device__ friend bool operator==(const linear_congruential_engine& l, const linear_congruential_engine& r) {
    return l.x_ == r.x_;
  }
  __host__ __device__ friend bool operator!=(const linear_congruential_engine& l, const linear_congruential_engine& r) {
    return l.x_ != r.x_;
  }

 private:
  result_type x_;
};
template <typename U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::multiplier;
template <typename U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::increment;
template <typename U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::modulus;
template <typename U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::min;
template <typename U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::max;
template <typename U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::default_seed;

// the 10000th draw of a default-constructed engine is 1043618065 / 399268537
typedef linear_congruential_engine<std::uint32_t, 16807, 0, 2147483647> minstd_rand0;
typedef linear_congruential_engine<std::uint32_t, 48271, 0, 2147483647> minstd_rand;
typedef minstd_rand default_random_engine;

// A real number in [a, b): the engine's draw, shifted to start at zero, over the number of values it can take.
template <typename RealType = double>
class uniform_real_distribution {
 public:
  typedef RealType result_type;
  typedef thrust::pair<RealType, RealType> param_type;
  __host__ __device__ explicit uniform_real_distribution(RealType a = 0.0, RealType b = 1.0) : param_(a, b) {}
  __host__ __device__ explicit uniform_real_distribution(const param_type& p) : param_(p) {}
  __host__ __device__ void reset() {}
  template <typename Engine>
  __host__ __device__ result_type operator()(Engine& urng) { return (*this)(urng, param_); }
  template <typename Engine>
  __host__ __device__ result_type operator()(Engine& urng, const param_type& p) {
    result_type result = static_cast<result_type>(urng() - Engine::min);
    result /= (result_type(1) + static_cast<result_type>(Engine::max - Engine::min));
    return (result * (p.second - p.first)) + p.first;
  }
  __host__ __device__ result_type a() const { return param_.first; }
  __host__ __device__ result_type b() const { return param_.second; }
  __host__ __device__ param_type param() const { return param_; }
  __host__ __device__ void param(const param_type& p) { param_ = p; }
  __host__ __device__ result_type min THRUST_AMD_NO_MACRO() const { return a(); }
  __host__ __device__ result_type max THRUST_AMD_NO_MACRO() const { return b(); }
  __host__ __device__ friend bool operator==(const uniform_real_distribution& l, const uniform_real_distribution& r) {
    return l.param_.first == r.param_.first && l.param_.second == r.param_.second;
  }
  __host__ __device__ friend bool operator!=(const uniform_real_distribution& l, const uniform_real_distribution& r) {
    return !(l == r);
  }

 private:
  param_type param_;
};

// An integer in [a, b]: a double in [a, b + 1), truncated.
template <typename IntType = int>
class uniform_int_distribution {
 public:
  typedef IntType result_type;
  typedef thrust::pair<IntType, IntType> param_type;
  __host__ __device__ explicit uniform_int_distribution(IntType a = 0, IntType b = std::numeric_limits<IntType>::max())
      : param_(a, b) {}
  __host__ __device__ explicit uniform_int_distribution(const param_type& p) : param_(p) {}
  __host__ __device__ void reset() {}
  template <typename Engine>
  __host__ __device__ result_type operator()(Engine& urng) { return (*this)(urng, param_); }
  template <typename Engine>
  __host__ __device__ result_type operator()(Engine& urng, const param_type& p) {
    uniform_real_distribution<double> real(static_cast<double>(p.first), static_cast<double>(p.second) + 1.0);
    return static_cast<result_type>(real(urng));
  }
  __host__ __device__ result_type a() const { return param_.first; }
  __host__ __device__ result_type b() const { return param_.second; }
  __host__ __device__ param_type param() const { return param_; }
  __host__ __device__ void param(const param_type& p) { param_ = p; }
  __host__ __device__ result_type min THRUST_AMD_NO_MACRO() const { return a(); }
  __host__ __device__ result_type max THRUST_AMD_NO_MACRO() const { return b(); }
  __host__ __device__ friend bool operator==(const uniform_int_distribution& l, const uniform_int_distribution& r) {
    return l.param_.first == r.param_.first && l.param_.second == r.param_.second;
  }
  __host__ __device__ friend bool operator!=(const uniform_int_distribution& l, const uniform_int_distribution& r) {
    return !(l == r);
  }

 private:
  param_type param_;
};

// Normal deviates two at a time from two uniform draws (the second one is kept for the next call).
template <typename RealType = double>
class normal_distribution {
 public:
  typedef RealType result_type;
  typedef thrust::pair<RealType, RealType> param_type;
  __host__ __device__ explicit normal_distribution(RealType mean = 0.0, RealType stddev = 1.0)
      : param_(mean, stddev), r1_(), r2_(), rho_(), valid_(false) {}
  __host__ __device__ explicit normal_distribution(const param_type& p)
      : param_(p), r1_(), r2_(), rho_(), valid_(false) {}
  __host__ __device__ void reset() { valid_ = false; }
  template <typename Engine>
  __host__ __device__ result_type operator()(Engine& urng) { return (*this)(urng, param_); }
  template <typename Engine>
  __host__ __device__ result_type operator()(Engine& urng, const param_type& p) {
    using std::cos;
    using std::log;
    using std::sin;
    using std::sqrt;
    if (!valid_) {
      uniform_real_distribution<RealType> u01;
      r1_ = u01(urng);
      r2_ = u01(urng);
      rho_ = sqrt(-RealType(2) * log(RealType(1) - r2_));
      valid_ = true;
    } else {
      valid_ = false;
    }
    const RealType pi = RealType(3.14159265358979323846);
    const RealType deviate = rho_ * (valid_ ? cos(RealType(2) * pi * r1_) : sin(RealType(2) * pi * r1_));
    return p.first + p.second * deviate;
  }
  __host__ __device__ result_type mean() const { return param_.first; }
  __host__ __device__ result_type stddev() const { return param_.second; }
  __host__ __device__ param_type param() const { return param_; }
  __host__ __device__ void param(const param_type& p) { param_ = p; }
  __host__ __device__ result_type min THRUST_AMD_NO_MACRO() const { return -std::numeric_limits<RealType>::max(); }
  __host__ __device__ result_type max THRUST_AMD_NO_MACRO() const { return std::numeric_limits<RealType>::max(); }
  __host__ __device__ friend bool operator==(const normal_distribution& l, const normal_distribution& r) {
    return l.param_.first == r.param_.first && l.param_.second == r.param_.second && l.valid_ == r.valid_ &&
           (!l.valid_ || (l.r1_ == r.r1_ && l.r2_ == r.r2_));
  }
  __host__ __device__ friend bool operator!=(const normal_distribution& l, const normal_distribution& r) {
    return !(l == r);
  }

 private:
  param_type param_;
  RealType r1_, r2_, rho_;
  bool valid_;
};

}  // namespace random

using random::default_random_engine;
using random::linear_congruential_engine;
using random::minstd_rand;
using random::minstd_rand0;
using random::normal_distribution;
using random::uniform_int_distribution;
using random::uniform_real_distribution;

}  // namespace thrust

