// Front-end test compiled with hipcc: thrust::random engines and distributions on the host and
// inside device code (testing/random.cu:237-352: the 10000th draw of minstd_rand0 and minstd_rand,
// discard against drawing, equality; :700-800 the distributions' ranges), and the common way of
// using them: one functor per element that seeds, discards and draws.
#include <thrust/device_vector.h>
#include <thrust/generate.h>
#include <thrust/host_vector.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/random.h>
#include <thrust/sequence.h>
#include <thrust/shuffle.h>
#include <thrust/sort.h>
#include <thrust/transform.h>
#include <thrust/transform_reduce.h>

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <sstream>

static int g_failed = 0, g_checks = 0;
static const char* g_test = "";
#define ASSERT_TRUE(c)                                                                    \
  do {                                                                                    \
    ++g_checks;                                                                           \
    if (!(c)) { ++g_failed; std::printf("FAIL [%s] %s:%d: %s\n", g_test, __FILE__, __LINE__, #c); } \
  } while (0)
#define ASSERT_EQUAL(a, b) ASSERT_TRUE((a) == (b))

// the 10000th draw of a default-constructed engine
template <typename Engine>
struct validate_engine {
  typename Engine::result_type value_10000;
  __host__ __device__ bool operator()() const {
    Engine e;
    e.discard(9999);
    return e() == value_10000;
  }
};
template <typename Engine>
struct validate_by_drawing {
  typename Engine::result_type value_10000;
  __host__ __device__ bool operator()() const {
    Engine e;
    typename Engine::result_type last = 0;
    for (int i = 0; i < 10000; ++i) last = e();
    return last == value_10000;
  }
};
template <typename Engine>
struct validate_discard_and_equality {
  __host__ __device__ bool operator()() const {
    Engine e0, e1;
    bool ok = e0 == e1;
    for (int i = 0; i < 10000; ++i) e0();
    ok &= e0 != e1;
    e1.discard(10000);
    ok &= e0 == e1;
    Engine e2(13), e3(13), e4(7);
    ok &= e2 == e3 && e2 != e4;
    e2.discard(5);
    ok &= e2 != e3;
    for (int i = 0; i < 5; ++i) e3();
    ok &= e2 == e3;
    // a seed that is a multiple of the modulus must not park the engine at zero
    Engine e5(Engine::modulus);
    ok &= e5() != 0;
    ok &= Engine::min == 1 && Engine::max == Engine::modulus - 1;
    return ok;
  }
};
template <typename Real>
struct validate_uniform_real {
  __host__ __device__ bool operator()() const {
    thrust::minstd_rand rng(17);
    thrust::uniform_real_distribution<Real> unit, wide(Real(-3), Real(9));
    bool ok = unit.a() == Real(0) && unit.b() == Real(1) && wide.min() == Real(-3) && wide.max() == Real(9);
    Real lo = Real(1), hi = Real(0);
    for (int i = 0; i < 20000; ++i) {
      const Real u = unit(rng), w = wide(rng);
      ok &= u >= Real(0) && u < Real(1) && w >= Real(-3) && w < Real(9);
      lo = u < lo ? u : lo;
      hi = u > hi ? u : hi;
    }
    return ok && lo < Real(0.01) && hi > Real(0.99);
  }
};
struct validate_uniform_int {
  __host__ __device__ bool operator()() const {
    thrust::default_random_engine rng(5);
    thrust::uniform_int_distribution<int> die(1, 6);
    bool ok = die.a() == 1 && die.b() == 6;
    int seen = 0;
    for (int i = 0; i < 5000; ++i) {
      const int v = die(rng);
      ok &= v >= 1 && v <= 6;
      seen |= 1 << v;
    }
    thrust::uniform_int_distribution<unsigned> coin(0u, 1u);
    for (int i = 0; i < 100; ++i) ok &= coin(rng) <= 1u;
    return ok && seen == 0x7e;
  }
};
// element i of a reproducible stream: seed, skip, draw
struct unit_draw {
  __host__ __device__ float operator()(unsigned long long i) const {
    thrust::default_random_engine rng(123);
    rng.discard(i);
    thrust::uniform_real_distribution<float> unit;
    return unit(rng);
  }
};
struct normal_draw {
  __host__ __device__ double operator()(unsigned long long i) const {
    thrust::minstd_rand rng(99);
    rng.discard(2 * i);
    thrust::normal_distribution<double> normal(10.0, 2.0);
    return normal(rng);
  }
};
struct squared_distance_from_ten {
  __host__ __device__ double operator()(double x) const { return (x - 10.0) * (x - 10.0); }
};

// what holds for any engine: discard against drawing, equality of equal histories, reseeding
template <typename Engine>
struct validate_histories {
  __host__ __device__ bool operator()() const {
    Engine e0, e1;
    bool ok = e0 == e1;
    for (int i = 0; i < 1000; ++i) e0();
    ok &= e0 != e1;
    e1.discard(1000);
    ok &= e0 == e1 && e0() == e1();
    Engine e2(13), e3(13), e4(7);
    ok &= e2 == e3 && e2 != e4 && e2() == e3();
    e4.seed(13);
    e4();
    ok &= e4 == e2;
    return ok;
  }
};

// written out after 10000 draws and read into an engine with another history: the same engine
// (testing/random.cu: the save / restore cases of every engine)
template <typename Engine>
static bool saves_and_restores() {
  Engine e0;
  e0.discard(10000);
  std::stringstream text;
  text << e0;
  Engine e1(7);
  e1.discard(3);
  text >> e1;
  return e0 == e1 && e0() == e1();
}

template <typename Vector, typename Check>
static bool holds_on(Check check) {
  Vector flag(1);
  thrust::generate(flag.begin(), flag.end(), check);
  return (bool)flag[0];
}

int main() {
  g_test = "engines";
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_engine<thrust::minstd_rand0>{1043618065u})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_engine<thrust::minstd_rand0>{1043618065u})));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_engine<thrust::minstd_rand>{399268537u})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_engine<thrust::minstd_rand>{399268537u})));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_by_drawing<thrust::minstd_rand0>{1043618065u})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_by_drawing<thrust::minstd_rand>{399268537u})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_by_drawing<thrust::default_random_engine>{399268537u})));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_discard_and_equality<thrust::minstd_rand0>())));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_discard_and_equality<thrust::minstd_rand0>())));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_discard_and_equality<thrust::minstd_rand>())));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_discard_and_equality<thrust::minstd_rand>())));
  // an engine with an increment and the natural modulus of its type: x <- 1664525 x + 1013904223 mod 2^32
  {
    thrust::linear_congruential_engine<std::uint32_t, 1664525u, 1013904223u, 0u> lcg(1);
    ASSERT_EQUAL(lcg(), 1015568748u);
    ASSERT_EQUAL(lcg(), 1586005467u);
    thrust::linear_congruential_engine<std::uint32_t, 1664525u, 1013904223u, 0u> skipped(1);
    skipped.discard(2);
    ASSERT_TRUE(skipped == lcg);
  }

  g_test = "the other engines";
  // the 10000th draw of each engine with predefined parameters (thrust/random.h:60-100,
  // thrust/random/subtract_with_carry_engine.h:225-245; testing/random.cu:237-360)
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_engine<thrust::ranlux24_base>{7937952u})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_engine<thrust::ranlux24_base>{7937952u})));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_engine<thrust::ranlux48_base>{192113843633948ull})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_engine<thrust::ranlux48_base>{192113843633948ull})));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_engine<thrust::ranlux24>{9901578u})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_engine<thrust::ranlux24>{9901578u})));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_engine<thrust::ranlux48>{88229545517833ull})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_engine<thrust::ranlux48>{88229545517833ull})));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_engine<thrust::taus88>{3535848941u})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_engine<thrust::taus88>{3535848941u})));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_by_drawing<thrust::ranlux24>{9901578u})));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_by_drawing<thrust::taus88>{3535848941u})));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_histories<thrust::ranlux24_base>())));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_histories<thrust::ranlux24_base>())));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_histories<thrust::ranlux48>())));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_histories<thrust::ranlux48>())));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_histories<thrust::taus88>())));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_histories<thrust::taus88>())));
  ASSERT_EQUAL(thrust::ranlux24_base::max, (1u << 24) - 1);
  ASSERT_EQUAL(thrust::ranlux48::max, (1ull << 48) - 1);
  ASSERT_EQUAL(thrust::taus88::min, 0u);

  g_test = "save and restore";
  ASSERT_TRUE(saves_and_restores<thrust::minstd_rand0>());
  ASSERT_TRUE(saves_and_restores<thrust::minstd_rand>());
  ASSERT_TRUE(saves_and_restores<thrust::ranlux24_base>());
  ASSERT_TRUE(saves_and_restores<thrust::ranlux48_base>());
  ASSERT_TRUE(saves_and_restores<thrust::ranlux24>());
  ASSERT_TRUE(saves_and_restores<thrust::ranlux48>());
  ASSERT_TRUE(saves_and_restores<thrust::taus88>());
  {
    std::stringstream text;
    text << thrust::uniform_real_distribution<float>(2.0f, 5.0f) << ' ' << thrust::uniform_int_distribution<int>(-3, 9) << ' '
         << thrust::normal_distribution<double>(1.5, 2.5);
    thrust::uniform_real_distribution<float> real;
    thrust::uniform_int_distribution<int> whole;
    thrust::normal_distribution<double> normal;
    text >> real >> whole >> normal;
    ASSERT_TRUE(real.a() == 2.0f && real.b() == 5.0f);
    ASSERT_TRUE(whole.a() == -3 && whole.b() == 9);
    ASSERT_TRUE(normal.mean() == 1.5 && normal.stddev() == 2.5);
  }

  g_test = "shuffle";
  {
    // every element once, and the copying form draws what the in-place form draws
    // (testing/shuffle.cu:327-360)
    thrust::device_vector<int> data(5), shuffled(5), again(5);
    thrust::sequence(data.begin(), data.end());
    shuffled = data;
    thrust::default_random_engine g(2);
    thrust::shuffle(shuffled.begin(), shuffled.end(), g);
    g.seed(2);
    thrust::shuffle_copy(data.begin(), data.end(), again.begin(), g);
    ASSERT_TRUE(shuffled == again);
    thrust::sort(shuffled.begin(), shuffled.end());
    ASSERT_TRUE(shuffled == data);
    // the permutation the reference draws for this generator (its CPP system, five elements, seed 2)
    const int drawn[] = {3, 0, 1, 2, 4};
    ASSERT_TRUE(again == thrust::host_vector<int>(drawn, drawn + 5));
    // the generator has moved on by the sixteen keys of the network
    thrust::default_random_engine sixteen(2);
    sixteen.discard(16);
    ASSERT_TRUE(g == sixteen);
  }
  for (size_t m : {size_t(0), size_t(1), size_t(2), size_t(3), size_t(31), size_t(32), size_t(33), size_t(1000), size_t(4097),
                   size_t(100000), size_t(1) << 20}) {
    // host and device draw the same permutation (testing/shuffle.cu:362-376), of any element type
    thrust::host_vector<long long> h(m);
    thrust::sequence(h.begin(), h.end());
    thrust::device_vector<long long> d(h);
    thrust::default_random_engine host_g(183), device_g(183);
    thrust::shuffle(h.begin(), h.end(), host_g);
    thrust::shuffle(d.begin(), d.end(), device_g);
    ASSERT_TRUE(d == h);
    ASSERT_TRUE(host_g == device_g);
    thrust::sort(d.begin(), d.end());
    bool every = true;
    thrust::host_vector<long long> sorted(d);
    for (size_t i = 0; i < m; ++i) every &= sorted[i] == (long long)i;
    ASSERT_TRUE(every);
    if (m > 32) {  // not the identity, and not the same for another seed
      thrust::host_vector<long long> other(m);
      thrust::sequence(other.begin(), other.end());
      thrust::default_random_engine other_g(184);
      thrust::shuffle(other.begin(), other.end(), other_g);
      ASSERT_TRUE(!(other == h));
      ASSERT_TRUE(!(sorted == h));
    }
  }
  {
    // the network is a bijection of [0, 2^bits) and knows its length (testing/shuffle.cu:378-425)
    thrust::default_random_engine g(0xD5);
    ASSERT_EQUAL(thrust::detail::cipher_domain(thrust::detail::make_index_cipher(3, g)), 4u);
    ASSERT_EQUAL(thrust::detail::cipher_domain(thrust::detail::make_index_cipher(2, g)), 2u);
    ASSERT_EQUAL(thrust::detail::cipher_domain(thrust::detail::make_index_cipher(0, g)), 1u);
    for (std::uint64_t m : {5ull, 64ull, 1000ull, 40000ull}) {
      thrust::default_random_engine host_g(0xD5), device_g(0xD5);
      const thrust::detail::image_under host_f = {thrust::detail::make_index_cipher(m, host_g)};
      const thrust::detail::image_under device_f = {thrust::detail::make_index_cipher(m, device_g)};
      const std::uint64_t n = thrust::detail::cipher_domain(host_f.cipher);
      thrust::host_vector<std::uint64_t> hr(n);
      thrust::device_vector<std::uint64_t> dr(n);
      thrust::sequence(hr.begin(), hr.end());
      thrust::sequence(dr.begin(), dr.end());
      thrust::transform(hr.begin(), hr.end(), hr.begin(), host_f);
      thrust::transform(dr.begin(), dr.end(), dr.begin(), device_f);
      ASSERT_TRUE(dr == hr);
      thrust::sort(dr.begin(), dr.end());
      thrust::host_vector<std::uint64_t> once(dr);
      bool every = true;
      for (std::uint64_t i = 0; i < n; ++i) every &= once[i] == i;
      ASSERT_TRUE(every);
    }
  }

  g_test = "distributions";
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_uniform_real<float>())));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_uniform_real<float>())));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_uniform_real<double>())));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_uniform_real<double>())));
  ASSERT_TRUE((holds_on<thrust::host_vector<bool> >(validate_uniform_int())));
  ASSERT_TRUE((holds_on<thrust::device_vector<bool> >(validate_uniform_int())));

  g_test = "one draw per element";
  const size_t n = 200000;
  thrust::counting_iterator<unsigned long long> index(0);
  thrust::host_vector<float> h(n);
  thrust::device_vector<float> d(n);
  thrust::transform(index, index + n, h.begin(), unit_draw());
  thrust::transform(index, index + n, d.begin(), unit_draw());
  thrust::host_vector<float> back = d;
  bool identical = true, in_range = true;
  double sum = 0;
  for (size_t i = 0; i < n; ++i) {
    identical &= back[i] == h[i];  // integer state, one division by a power of two: the same on both sides
    in_range &= h[i] >= 0.0f && h[i] < 1.0f;
    sum += h[i];
  }
  ASSERT_TRUE(identical);
  ASSERT_TRUE(in_range);
  ASSERT_TRUE(std::fabs(sum / n - 0.5) < 0.01);
  // the stream element by element equals one engine drawn n times
  {
    thrust::default_random_engine rng(123);
    thrust::uniform_real_distribution<float> unit;
    bool same_stream = true;
    for (size_t i = 0; i < 1000; ++i) same_stream &= unit(rng) == h[i];
    ASSERT_TRUE(same_stream);
  }
  thrust::host_vector<double> hn(n);
  thrust::device_vector<double> dn(n);
  thrust::transform(index, index + n, hn.begin(), normal_draw());
  thrust::transform(index, index + n, dn.begin(), normal_draw());
  thrust::host_vector<double> backn = dn;
  bool close = true;
  for (size_t i = 0; i < n; ++i) close &= std::fabs(backn[i] - hn[i]) <= 1e-9 * (1.0 + std::fabs(hn[i]));
  ASSERT_TRUE(close);  // log, sqrt, cos of the two math libraries agree to rounding
  const double mean = thrust::reduce(dn.begin(), dn.end(), 0.0) / n;
  const double var = thrust::transform_reduce(dn.begin(), dn.end(), squared_distance_from_ten(), 0.0, thrust::plus<double>()) / n;
  ASSERT_TRUE(std::fabs(mean - 10.0) < 0.05);
  ASSERT_TRUE(std::fabs(var - 4.0) < 0.1);

  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
