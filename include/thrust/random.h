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
#include <type_traits>

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

  // the state as text, and back (thrust/random/detail/*_engine.inl: stream_out / stream_in)
  template <typename CharT, typename Traits>
  friend std::basic_ostream<CharT, Traits>& operator<<(std::basic_ostream<CharT, Traits>& os, const linear_congruential_engine& e) {
    const typename std::basic_ostream<CharT, Traits>::fmtflags flags = os.flags();
    const CharT fill = os.fill();
    os.flags(std::ios_base::dec | std::ios_base::fixed | std::ios_base::left);
    os.fill(os.widen(' '));
    os << e.x_;
    os.flags(flags);
    os.fill(fill);
    return os;
  }
  template <typename CharT, typename Traits>
  friend std::basic_istream<CharT, Traits>& operator>>(std::basic_istream<CharT, Traits>& is, linear_congruential_engine& e) {
    const typename std::basic_istream<CharT, Traits>::fmtflags flags = is.flags();
    is.flags(std::ios_base::dec | std::ios_base::skipws);
    is >> e.x_;
    is.flags(flags);
    return is;
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

// ------------------------------------------------------------------ the other engines
// A Tausworthe generator (thrust/random/linear_feedback_shift_engine.h:50-200,
// detail/linear_feedback_shift_engine.inl:27-60).
template <typename UIntType, std::size_t w, std::size_t k, std::size_t q, std::size_t s>
class linear_feedback_shift_engine {
 public:
  typedef UIntType result_type;
  static const std::size_t word_size = w, exponent1 = k, exponent2 = q, step_size = s;
  // bits 1 .. w-1: the mask the reference builds leaves bit 0 out
  // (random/detail/linear_feedback_shift_engine_wordmask.h:27-40), and the validation value of
  // taus88 is the one this mask gives
  static const result_type wordmask =
      (result_type)((w < 8 * sizeof(UIntType) ? (result_type)((result_type)1 << (w % (8 * sizeof(UIntType)))) : (result_type)0) - 2);
  static const result_type min = 0;
  static const result_type max = wordmask;
  static const result_type default_seed = 341u;

  __host__ __device__ explicit linear_feedback_shift_engine(result_type value = default_seed) { seed(value); }
  __host__ __device__ void seed(result_type value = default_seed) { x_ = value; }
  __host__ __device__ result_type operator()() {
    const UIntType b = (UIntType)((((x_ << q) ^ x_) & wordmask) >> (k - s));
    const UIntType mask = (UIntType)(((~static_cast<UIntType>(0)) << (w - k)) & wordmask);
    x_ = (UIntType)(((x_ & mask) << s) ^ b);
    return x_;
  }
  __host__ __device__ void discard(unsigned long long z) {
    for (; z > 0; --z) (*this)();
  }
  __host__ __device__ friend bool operator==(const linear_feedback_shift_engine& a, const linear_feedback_shift_engine& b) {
    return a.x_ == b.x_;
  }
  __host__ __device__ friend bool operator!=(const linear_feedback_shift_engine& a, const linear_feedback_shift_engine& b) {
    return !(a == b);
  }

  // the state as text, and back (thrust/random/detail/*_engine.inl: stream_out / stream_in)
  template <typename CharT, typename Traits>
  friend std::basic_ostream<CharT, Traits>& operator<<(std::basic_ostream<CharT, Traits>& os, const linear_feedback_shift_engine& e) {
    const typename std::basic_ostream<CharT, Traits>::fmtflags flags = os.flags();
    const CharT fill = os.fill();
    os.flags(std::ios_base::dec | std::ios_base::fixed | std::ios_base::left);
    os.fill(os.widen(' '));
    os << e.x_;
    os.flags(flags);
    os.fill(fill);
    return os;
  }
  template <typename CharT, typename Traits>
  friend std::basic_istream<CharT, Traits>& operator>>(std::basic_istream<CharT, Traits>& is, linear_feedback_shift_engine& e) {
    const typename std::basic_istream<CharT, Traits>::fmtflags flags = is.flags();
    is.flags(std::ios_base::dec | std::ios_base::skipws);
    is >> e.x_;
    is.flags(flags);
    return is;
  }
 private:
  result_type x_;
};
template <typename U, std::size_t w, std::size_t k, std::size_t q, std::size_t s>
const U linear_feedback_shift_engine<U, w, k, q, s>::wordmask;
template <typename U, std::size_t w, std::size_t k, std::size_t q, std::size_t s>
const U linear_feedback_shift_engine<U, w, k, q, s>::min;
template <typename U, std::size_t w, std::size_t k, std::size_t q, std::size_t s>
const U linear_feedback_shift_engine<U, w, k, q, s>::max;
template <typename U, std::size_t w, std::size_t k, std::size_t q, std::size_t s>
const U linear_feedback_shift_engine<U, w, k, q, s>::default_seed;

// x_i = (x_{i-s} - x_{i-r} - carry) mod 2^w (thrust/random/subtract_with_carry_engine.h:55-215,
// detail/subtract_with_carry_engine.inl:30-85).  The r words of state are seeded with one draw
// each of a 40014 / 2147483563 congruential engine, which is the reference's rule (and not the
// C++ standard's, whose engines of the same names give other numbers).
template <typename UIntType, std::size_t w, std::size_t s, std::size_t r>
class subtract_with_carry_engine {
 public:
  typedef UIntType result_type;
  static const std::size_t word_size = w, short_lag = s, long_lag = r;
  static const result_type modulus = (result_type)((result_type)1 << w);
  static const result_type min = 0;
  static const result_type max = modulus - 1;
  static const result_type default_seed = 19780503u;

  __host__ __device__ explicit subtract_with_carry_engine(result_type value = default_seed) { seed(value); }
  __host__ __device__ void seed(result_type value = default_seed) {
    linear_congruential_engine<result_type, 40014u, 0u, 2147483563u> e(value == 0u ? (result_type)default_seed : value);
    for (std::size_t i = 0; i < r; ++i) x_[i] = (result_type)(e() % modulus);
    carry_ = x_[r - 1] == 0;
    k_ = 0;
  }
  __host__ __device__ result_type operator()() {
    int short_index = k_ - (int)s;
    if (short_index < 0) short_index += (int)r;
    result_type xi;
    if (x_[short_index] >= x_[k_] + carry_) {
      xi = x_[short_index] - x_[k_] - carry_;
      carry_ = 0;
    } else {
      xi = modulus - x_[k_] - carry_ + x_[short_index];
      carry_ = 1;
    }
    x_[k_] = xi;
    if (++k_ >= (int)r) k_ = 0;
    return xi;
  }
  __host__ __device__ void discard(unsigned long long z) {
    for (; z > 0; --z) (*this)();
  }
  // the same future: the same words in the same order from where each one stands, and the same carry
  __host__ __device__ friend bool operator==(const subtract_with_carry_engine& a, const subtract_with_carry_engine& b) {
    bool same = a.carry_ == b.carry_;
    for (std::size_t i = 0; i < r; ++i) same = same && a.x_[(i + a.k_) % r] == b.x_[(i + b.k_) % r];
    return same;
  }
  __host__ __device__ friend bool operator!=(const subtract_with_carry_engine& a, const subtract_with_carry_engine& b) {
    return !(a == b);
  }

  // the state as text, and back (thrust/random/detail/*_engine.inl: stream_out / stream_in)
  template <typename CharT, typename Traits>
  friend std::basic_ostream<CharT, Traits>& operator<<(std::basic_ostream<CharT, Traits>& os, const subtract_with_carry_engine& e) {
    const typename std::basic_ostream<CharT, Traits>::fmtflags flags = os.flags();
    const CharT fill = os.fill();
    os.flags(std::ios_base::dec | std::ios_base::fixed | std::ios_base::left);
    os.fill(os.widen(' '));
    for (std::size_t i = 0; i < r; ++i) os << e.x_[(i + e.k_) % r] << os.widen(' ');
    os << e.carry_;
    os.flags(flags);
    os.fill(fill);
    return os;
  }
  template <typename CharT, typename Traits>
  friend std::basic_istream<CharT, Traits>& operator>>(std::basic_istream<CharT, Traits>& is, subtract_with_carry_engine& e) {
    const typename std::basic_istream<CharT, Traits>::fmtflags flags = is.flags();
    is.flags(std::ios_base::dec | std::ios_base::skipws);
    for (std::size_t i = 0; i < r; ++i) is >> e.x_[i];
    is >> e.carry_;
    e.k_ = 0;
    is.flags(flags);
    return is;
  }
 private:
  result_type x_[r];
  result_type carry_;
  int k_;
};
template <typename U, std::size_t w, std::size_t s, std::size_t r> const U subtract_with_carry_engine<U, w, s, r>::modulus;
template <typename U, std::size_t w, std::size_t s, std::size_t r> const U subtract_with_carry_engine<U, w, s, r>::min;
template <typename U, std::size_t w, std::size_t s, std::size_t r> const U subtract_with_carry_engine<U, w, s, r>::max;
template <typename U, std::size_t w, std::size_t s, std::size_t r> const U subtract_with_carry_engine<U, w, s, r>::default_seed;

// Of every p draws of Engine the first r (thrust/random/discard_block_engine.h:45-200,
// detail/discard_block_engine.inl:27-90).
template <typename Engine, std::size_t p, std::size_t r>
class discard_block_engine {
 public:
  typedef Engine base_type;
  typedef typename base_type::result_type result_type;
  static const std::size_t block_size = p, used_block = r;
  static const result_type min = base_type::min;
  static const result_type max = base_type::max;

  __host__ __device__ discard_block_engine() : e_(), n_(0) {}
  __host__ __device__ explicit discard_block_engine(result_type s) : e_(s), n_(0) {}
  __host__ __device__ explicit discard_block_engine(const base_type& urng) : e_(urng), n_(0) {}
  __host__ __device__ void seed() { e_.seed(); n_ = 0; }
  __host__ __device__ void seed(result_type s) { e_.seed(s); n_ = 0; }
  __host__ __device__ result_type operator()() {
    if (n_ >= r) {
      e_.discard(p - n_);
      n_ = 0;
    }
    ++n_;
    return e_();
  }
  __host__ __device__ void discard(unsigned long long z) {
    for (; z > 0; --z) (*this)();
  }
  __host__ __device__ const base_type& base() const { return e_; }
  __host__ __device__ friend bool operator==(const discard_block_engine& a, const discard_block_engine& b) {
    return a.e_ == b.e_ && a.n_ == b.n_;
  }
  __host__ __device__ friend bool operator!=(const discard_block_engine& a, const discard_block_engine& b) { return !(a == b); }

  // the state as text, and back (thrust/random/detail/*_engine.inl: stream_out / stream_in)
  template <typename CharT, typename Traits>
  friend std::basic_ostream<CharT, Traits>& operator<<(std::basic_ostream<CharT, Traits>& os, const discard_block_engine& e) {
    const typename std::basic_ostream<CharT, Traits>::fmtflags flags = os.flags();
    const CharT fill = os.fill();
    os.flags(std::ios_base::dec | std::ios_base::fixed | std::ios_base::left);
    os.fill(os.widen(' '));
    os << e.e_ << os.widen(' ') << e.n_;
    os.flags(flags);
    os.fill(fill);
    return os;
  }
  template <typename CharT, typename Traits>
  friend std::basic_istream<CharT, Traits>& operator>>(std::basic_istream<CharT, Traits>& is, discard_block_engine& e) {
    const typename std::basic_istream<CharT, Traits>::fmtflags flags = is.flags();
    is.flags(std::ios_base::dec | std::ios_base::skipws);
    is >> e.e_ >> e.n_;
    is.flags(flags);
    return is;
  }
 private:
  base_type e_;
  unsigned int n_;
};
template <typename E, std::size_t p, std::size_t r> const typename E::result_type discard_block_engine<E, p, r>::min;
template <typename E, std::size_t p, std::size_t r> const typename E::result_type discard_block_engine<E, p, r>::max;

// The draws of two engines, shifted and combined by exclusive or
// (thrust/random/xor_combine_engine.h:50-230, detail/xor_combine_engine.inl:27-120).
template <typename Engine1, std::size_t s1, typename Engine2, std::size_t s2 = 0u>
class xor_combine_engine {
 public:
  typedef Engine1 base1_type;
  typedef Engine2 base2_type;
  typedef typename std::conditional<(sizeof(typename base2_type::result_type) > sizeof(typename base1_type::result_type)),
                                    typename base2_type::result_type, typename base1_type::result_type>::type result_type;
  static const std::size_t shift1 = s1, shift2 = s2;
  static const result_type min = 0;

 private:
  // all ones up to the highest bit either side can set: the exact bound for the engines whose
  // ranges end one below a power of two or, as taus88's parts do, two below
  static constexpr result_type ones_up_to(result_type x) {
    return x == 0 ? 0 : (result_type)(ones_up_to((result_type)(x >> 1)) << 1 | 1);
  }

 public:
  static const result_type max = ones_up_to((result_type)(((result_type)(base1_type::max - base1_type::min) << s1) |
                                                           ((result_type)(base2_type::max - base2_type::min) << s2)));

  __host__ __device__ xor_combine_engine() : b1_(), b2_() {}
  __host__ __device__ xor_combine_engine(const base1_type& urng1, const base2_type& urng2) : b1_(urng1), b2_(urng2) {}
  __host__ __device__ explicit xor_combine_engine(result_type s) : b1_(s), b2_(s) {}
  __host__ __device__ void seed() { b1_.seed(); b2_.seed(); }
  __host__ __device__ void seed(result_type s) { b1_.seed(s); b2_.seed(s); }
  __host__ __device__ const base1_type& base1() const { return b1_; }
  __host__ __device__ const base2_type& base2() const { return b2_; }
  __host__ __device__ result_type operator()() {
    return (result_type)((result_type(b1_() - base1_type::min) << shift1) ^ (result_type(b2_() - base2_type::min) << shift2));
  }
  __host__ __device__ void discard(unsigned long long z) {
    for (; z > 0; --z) (*this)();
  }
  __host__ __device__ friend bool operator==(const xor_combine_engine& a, const xor_combine_engine& b) {
    return a.b1_ == b.b1_ && a.b2_ == b.b2_;
  }
  __host__ __device__ friend bool operator!=(const xor_combine_engine& a, const xor_combine_engine& b) { return !(a == b); }

  // the state as text, and back (thrust/random/detail/*_engine.inl: stream_out / stream_in)
  template <typename CharT, typename Traits>
  friend std::basic_ostream<CharT, Traits>& operator<<(std::basic_ostream<CharT, Traits>& os, const xor_combine_engine& e) {
    const typename std::basic_ostream<CharT, Traits>::fmtflags flags = os.flags();
    const CharT fill = os.fill();
    os.flags(std::ios_base::dec | std::ios_base::fixed | std::ios_base::left);
    os.fill(os.widen(' '));
    os << e.b1_ << os.widen(' ') << e.b2_;
    os.flags(flags);
    os.fill(fill);
    return os;
  }
  template <typename CharT, typename Traits>
  friend std::basic_istream<CharT, Traits>& operator>>(std::basic_istream<CharT, Traits>& is, xor_combine_engine& e) {
    const typename std::basic_istream<CharT, Traits>::fmtflags flags = is.flags();
    is.flags(std::ios_base::dec | std::ios_base::skipws);
    is >> e.b1_ >> e.b2_;
    is.flags(flags);
    return is;
  }
 private:
  base1_type b1_;
  base2_type b2_;
};
template <typename E1, std::size_t s1, typename E2, std::size_t s2>
const typename xor_combine_engine<E1, s1, E2, s2>::result_type xor_combine_engine<E1, s1, E2, s2>::min;
template <typename E1, std::size_t s1, typename E2, std::size_t s2>
const typename xor_combine_engine<E1, s1, E2, s2>::result_type xor_combine_engine<E1, s1, E2, s2>::max;

// The engines with predefined parameters and the 10000th draw of a default-constructed one
// (thrust/random.h:60-100, subtract_with_carry_engine.h:225-245): ranlux24_base 7937952,
// ranlux48_base 192113843633948, ranlux24 9901578, ranlux48 88229545517833, taus88 3535848941.
typedef subtract_with_carry_engine<std::uint32_t, 24, 10, 24> ranlux24_base;
typedef subtract_with_carry_engine<std::uint64_t, 48, 5, 12> ranlux48_base;
typedef discard_block_engine<ranlux24_base, 223, 23> ranlux24;
typedef discard_block_engine<ranlux48_base, 389, 11> ranlux48;
typedef xor_combine_engine<linear_feedback_shift_engine<std::uint32_t, 32u, 31u, 13u, 12u>, 0,
                           xor_combine_engine<linear_feedback_shift_engine<std::uint32_t, 32u, 29u, 2u, 4u>, 0,
                                              linear_feedback_shift_engine<std::uint32_t, 32u, 28u, 3u, 17u>, 0>,
                           0>
    taus88;

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

  // the parameters as text, and back (the two parameters)
  template <typename CharT, typename Traits>
  friend std::basic_ostream<CharT, Traits>& operator<<(std::basic_ostream<CharT, Traits>& os, const uniform_real_distribution& e) {
    const typename std::basic_ostream<CharT, Traits>::fmtflags flags = os.flags();
    const CharT fill = os.fill();
    os.flags(std::ios_base::dec | std::ios_base::fixed | std::ios_base::left);
    os.fill(os.widen(' '));
    os << e.param_.first << os.widen(' ') << e.param_.second;
    os.flags(flags);
    os.fill(fill);
    return os;
  }
  template <typename CharT, typename Traits>
  friend std::basic_istream<CharT, Traits>& operator>>(std::basic_istream<CharT, Traits>& is, uniform_real_distribution& e) {
    const typename std::basic_istream<CharT, Traits>::fmtflags flags = is.flags();
    is.flags(std::ios_base::dec | std::ios_base::skipws);
    is >> e.param_.first >> e.param_.second;
    is.flags(flags);
    return is;
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

  // the parameters as text, and back (the two parameters)
  template <typename CharT, typename Traits>
  friend std::basic_ostream<CharT, Traits>& operator<<(std::basic_ostream<CharT, Traits>& os, const uniform_int_distribution& e) {
    const typename std::basic_ostream<CharT, Traits>::fmtflags flags = os.flags();
    const CharT fill = os.fill();
    os.flags(std::ios_base::dec | std::ios_base::fixed | std::ios_base::left);
    os.fill(os.widen(' '));
    os << e.param_.first << os.widen(' ') << e.param_.second;
    os.flags(flags);
    os.fill(fill);
    return os;
  }
  template <typename CharT, typename Traits>
  friend std::basic_istream<CharT, Traits>& operator>>(std::basic_istream<CharT, Traits>& is, uniform_int_distribution& e) {
    const typename std::basic_istream<CharT, Traits>::fmtflags flags = is.flags();
    is.flags(std::ios_base::dec | std::ios_base::skipws);
    is >> e.param_.first >> e.param_.second;
    is.flags(flags);
    return is;
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

  // the parameters as text, and back (mean and standard deviation)
  template <typename CharT, typename Traits>
  friend std::basic_ostream<CharT, Traits>& operator<<(std::basic_ostream<CharT, Traits>& os, const normal_distribution& e) {
    const typename std::basic_ostream<CharT, Traits>::fmtflags flags = os.flags();
    const CharT fill = os.fill();
    os.flags(std::ios_base::dec | std::ios_base::fixed | std::ios_base::left);
    os.fill(os.widen(' '));
    os << e.param_.first << os.widen(' ') << e.param_.second;
    os.flags(flags);
    os.fill(fill);
    return os;
  }
  template <typename CharT, typename Traits>
  friend std::basic_istream<CharT, Traits>& operator>>(std::basic_istream<CharT, Traits>& is, normal_distribution& e) {
    const typename std::basic_istream<CharT, Traits>::fmtflags flags = is.flags();
    is.flags(std::ios_base::dec | std::ios_base::skipws);
    is >> e.param_.first >> e.param_.second;
    is.flags(flags);
    return is;
  }
 private:
  param_type param_;
  RealType r1_, r2_, rho_;
  bool valid_;
};

}  // namespace random

using random::default_random_engine;
using random::discard_block_engine;
using random::linear_feedback_shift_engine;
using random::ranlux24;
using random::ranlux24_base;
using random::ranlux48;
using random::ranlux48_base;
using random::subtract_with_carry_engine;
using random::taus88;
using random::xor_combine_engine;
using random::linear_congruential_engine;
using random::minstd_rand;
using random::minstd_rand0;
using random::normal_distribution;
using random::uniform_int_distribution;
using random::uniform_real_distribution;

}  // namespace thrust

