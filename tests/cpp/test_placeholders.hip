// Front-end test compiled with hipcc: placeholder expressions as functors of the device
// system's algorithms, as the reference's unit tests use them
// (testing/functional_placeholders_arithmetic.cu:6-80, _bitwise.cu, _logical.cu,
// _relational.cu, _compound_assignment.cu:6-191, _miscellaneous.cu:18-62,
// inner_product.cu: TestInnerProductPlaceholders).  Every expression runs through
// thrust::transform on host_vector and on device_vector and is compared with the same
// operation written out as a loop.
#include <thrust/copy.h>
#include <thrust/count.h>
#include <thrust/device_vector.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/inner_product.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/partition.h>
#include <thrust/reduce.h>
#include <thrust/transform.h>

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <vector>

static int g_failed = 0, g_checks = 0;
static const char* g_test = "";
#define ASSERT_TRUE(c)                                                                    \
  do {                                                                                    \
    ++g_checks;                                                                           \
    if (!(c)) { ++g_failed; std::printf("FAIL [%s] %s:%d: %s\n", g_test, __FILE__, __LINE__, #c); } \
  } while (0)

static uint64_t mix(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
template <typename T>
static thrust::host_vector<T> samples(size_t n, uint64_t seed) {
  thrust::host_vector<T> h(n);
  for (size_t i = 0; i < n; ++i) h[i] = (T)((int)(mix(seed * 1000003ull + i) % 200) - (std::is_signed<T>::value ? 100 : 0));
  return h;
}
template <typename A, typename B>
static bool same(const A& a, const B& b) {
  if (a.size() != b.size()) return false;
  for (size_t i = 0; i < a.size(); ++i)
    if (!(a[i] == b[i])) return false;
  return true;
}

static const size_t kN = 10000;

// result[i] = expr(lhs[i], rhs[i]) on both systems against the loop `reference`
template <typename T, typename R, typename Expr, typename Ref>
static void binary_case(const char* what, Expr expr, Ref reference, bool nonzero_rhs) {
  g_test = what;
  thrust::host_vector<T> lhs = samples<T>(kN, 1), rhs = samples<T>(kN, 2);
  if (nonzero_rhs)
    for (size_t i = 0; i < kN; ++i)
      if (rhs[i] == T(0)) rhs[i] = T(1);
  std::vector<R> expect(kN);
  for (size_t i = 0; i < kN; ++i) expect[i] = (R)reference(lhs[i], rhs[i]);
  thrust::host_vector<R> h_result(kN);
  thrust::transform(lhs.begin(), lhs.end(), rhs.begin(), h_result.begin(), expr);
  ASSERT_TRUE(same(h_result, expect));
  thrust::device_vector<T> d_lhs = lhs, d_rhs = rhs;
  thrust::device_vector<R> d_result(kN);
  thrust::transform(d_lhs.begin(), d_lhs.end(), d_rhs.begin(), d_result.begin(), expr);
  ASSERT_TRUE(same(thrust::host_vector<R>(d_result), expect));
}
template <typename T, typename R, typename Expr, typename Ref>
static void unary_case(const char* what, Expr expr, Ref reference, bool nonzero) {
  g_test = what;
  thrust::host_vector<T> in = samples<T>(kN, 3);
  if (nonzero)
    for (size_t i = 0; i < kN; ++i)
      if (in[i] == T(0)) in[i] = T(1);
  std::vector<R> expect(kN);
  for (size_t i = 0; i < kN; ++i) expect[i] = (R)reference(in[i]);
  thrust::host_vector<R> h_result(kN);
  thrust::transform(in.begin(), in.end(), h_result.begin(), expr);
  ASSERT_TRUE(same(h_result, expect));
  thrust::device_vector<T> d_in = in;
  thrust::device_vector<R> d_result(kN);
  thrust::transform(d_in.begin(), d_in.end(), d_result.begin(), expr);
  ASSERT_TRUE(same(thrust::host_vector<R>(d_result), expect));
}

#define BINARY(T, R, OP, NONZERO)                                                                         \
  binary_case<T, R>("_1 " #OP " _2 <" #T ">", _1 OP _2, [](T a, T b) { return a OP b; }, NONZERO);          \
  unary_case<T, R>("_1 " #OP " T(1) <" #T ">", _1 OP T(1), [](T a) { return a OP T(1); }, false);           \
  unary_case<T, R>("T(1) " #OP " _1 <" #T ">", T(1) OP _1, [](T a) { return T(1) OP a; }, NONZERO);

template <typename T>
static void Arithmetic() {
  using namespace thrust::placeholders;
  BINARY(T, T, +, false)
  BINARY(T, T, -, false)
  BINARY(T, T, *, false)
  BINARY(T, T, /, true)
  unary_case<T, T>("+_1", +_1, [](T a) { return (T)(+a); }, false);
  unary_case<T, T>("-_1", -_1, [](T a) { return (T)(-a); }, false);
  // saxpy with a captured value (functional_placeholders_miscellaneous.cu:18-40)
  const T a(13);
  binary_case<T, T>("a * _1 + _2", a * _1 + _2, [](T x, T y) { return T(13) * x + y; }, false);
  binary_case<T, T>("(_1 + _2) * (_1 - _2)", (_1 + _2) * (_1 - _2), [](T x, T y) { return (x + y) * (x - y); }, false);
}
template <typename T>
static void IntegralOnly() {
  using namespace thrust::placeholders;
  BINARY(T, T, %, true)
  BINARY(T, T, &, false)
  BINARY(T, T, |, false)
  BINARY(T, T, ^, false)
  unary_case<T, T>("~_1", ~_1, [](T a) { return (T)(~a); }, false);
  unary_case<T, T>("_1 << 2", _1 << 2, [](T a) { return (T)(a << 2); }, false);
  unary_case<T, T>("_1 >> 1", _1 >> 1, [](T a) { return (T)(a >> 1); }, false);
}
template <typename T>
static void LogicalAndRelational() {
  using namespace thrust::placeholders;
  BINARY(T, bool, &&, false)
  BINARY(T, bool, ||, false)
  BINARY(T, bool, ==, false)
  BINARY(T, bool, !=, false)
  BINARY(T, bool, <, false)
  BINARY(T, bool, >, false)
  BINARY(T, bool, <=, false)
  BINARY(T, bool, >=, false)
  unary_case<T, bool>("!_1", !_1, [](T a) { return !a; }, false);
  unary_case<T, bool>("_1 > 2 && _1 < 50", _1 > T(2) && _1 < T(50), [](T a) { return a > T(2) && a < T(50); }, false);
}

// Compound assignment writes through the first argument and yields its new value
// (functional_placeholders_compound_assignment.cu:6-191).
#define COMPOUND(T, OP, NONZERO)                                                                            \
  {                                                                                                         \
    g_test = "_1 " #OP " _2 <" #T ">";                                                                      \
    thrust::host_vector<T> lhs = samples<T>(kN, 4), rhs = samples<T>(kN, 5);                                \
    if (NONZERO)                                                                                            \
      for (size_t i = 0; i < kN; ++i)                                                                       \
        if (rhs[i] == T(0)) rhs[i] = T(1);                                                                  \
    std::vector<T> expect_lhs(lhs.begin(), lhs.end()), expect(kN);                                          \
    for (size_t i = 0; i < kN; ++i) expect[i] = (expect_lhs[i] OP rhs[i]);                                  \
    thrust::device_vector<T> d_lhs = lhs, d_rhs = rhs, d_result(kN);                                        \
    thrust::host_vector<T> h_lhs = lhs, h_result(kN);                                                       \
    thrust::transform(h_lhs.begin(), h_lhs.end(), rhs.begin(), h_result.begin(), _1 OP _2);                 \
    thrust::transform(d_lhs.begin(), d_lhs.end(), d_rhs.begin(), d_result.begin(), _1 OP _2);               \
    ASSERT_TRUE(same(h_result, expect));                                                                    \
    ASSERT_TRUE(same(h_lhs, expect_lhs));                                                                   \
    ASSERT_TRUE(same(thrust::host_vector<T>(d_result), expect));                                            \
    ASSERT_TRUE(same(thrust::host_vector<T>(d_lhs), expect_lhs));                                           \
  }

template <typename T>
static void CompoundAssignment() {
  using namespace thrust::placeholders;
  COMPOUND(T, +=, false)
  COMPOUND(T, -=, false)
  COMPOUND(T, *=, false)
  COMPOUND(T, /=, true)
}
template <typename T>
static void CompoundAssignmentIntegral() {
  using namespace thrust::placeholders;
  COMPOUND(T, %=, true)
  COMPOUND(T, &=, false)
  COMPOUND(T, |=, false)
  COMPOUND(T, ^=, false)
  // prefix and suffix increment / decrement: the element changes, the result is the new / the old value
  g_test = "++_1, _1++, --_1, _1--";
  thrust::host_vector<T> in = samples<T>(kN, 6);
  for (int form = 0; form < 4; ++form) {
    thrust::device_vector<T> d_in = in, d_result(kN);
    std::vector<T> expect_in(in.begin(), in.end()), expect(kN);
    for (size_t i = 0; i < kN; ++i)
      expect[i] = form == 0 ? ++expect_in[i] : form == 1 ? expect_in[i]++ : form == 2 ? --expect_in[i] : expect_in[i]--;
    if (form == 0) thrust::transform(d_in.begin(), d_in.end(), d_result.begin(), ++_1);
    if (form == 1) thrust::transform(d_in.begin(), d_in.end(), d_result.begin(), _1++);
    if (form == 2) thrust::transform(d_in.begin(), d_in.end(), d_result.begin(), --_1);
    if (form == 3) thrust::transform(d_in.begin(), d_in.end(), d_result.begin(), _1--);
    ASSERT_TRUE(same(thrust::host_vector<T>(d_result), expect));
    ASSERT_TRUE(same(thrust::host_vector<T>(d_in), expect_in));
  }
}

static void TestPlaceholdersInOtherAlgorithms() {
  using namespace thrust::placeholders;
  g_test = "InnerProductPlaceholders";
  {
    thrust::device_vector<float> v1(100, 1.f), v2(100, 1.f);
    auto result = thrust::inner_product(v1.begin(), v1.end(), v2.begin(), 0.0f, thrust::plus<float>{}, _1 * _2 + 1.0f);
    ASSERT_TRUE(std::fabs(result - 200.f) < 1e-3f);
  }
  g_test = "FunctionalPlaceholdersTransformIterator";
  {
    const int a = 13;
    thrust::host_vector<int> x = samples<int>(kN, 7), y = samples<int>(kN, 8);
    thrust::device_vector<int> dx = x, dy = y, result(kN);
    thrust::transform(thrust::make_transform_iterator(dx.begin(), a * _1), thrust::make_transform_iterator(dx.end(), a * _1),
                      dy.begin(), result.begin(), _1 + _2);
    std::vector<int> expect(kN);
    for (size_t i = 0; i < kN; ++i) expect[i] = a * x[i] + y[i];
    ASSERT_TRUE(same(thrust::host_vector<int>(result), expect));
  }
  g_test = "placeholder predicates in count_if / copy_if / partition / reduce";
  {
    thrust::host_vector<int> h = samples<int>(kN, 9);
    thrust::device_vector<int> d = h, out(kN);
    // `_1 CMP value` stays the library's own predicate form; compound predicates are kernels of their own
    const size_t below = (size_t)std::count_if(h.begin(), h.end(), [](int v) { return v < 10; });
    ASSERT_TRUE((size_t)thrust::count_if(d.begin(), d.end(), _1 < 10) == below);
    ASSERT_TRUE((size_t)thrust::count_if(d.begin(), d.end(), 10 > _1) == below);
    const size_t between = (size_t)std::count_if(h.begin(), h.end(), [](int v) { return v > -20 && v % 3 == 0; });
    ASSERT_TRUE((size_t)thrust::count_if(d.begin(), d.end(), _1 > -20 && _1 % 3 == 0) == between);
    auto end = thrust::copy_if(d.begin(), d.end(), out.begin(), _1 > -20 && _1 % 3 == 0);
    ASSERT_TRUE((size_t)(end - out.begin()) == between);
    std::vector<int> expect;
    for (size_t i = 0; i < kN; ++i)
      if (h[i] > -20 && h[i] % 3 == 0) expect.push_back(h[i]);
    out.resize(between);
    ASSERT_TRUE(same(thrust::host_vector<int>(out), expect));
    auto mid = thrust::stable_partition(d.begin(), d.end(), (_1 & 1) == 0);
    const size_t evens = (size_t)std::count_if(h.begin(), h.end(), [](int v) { return (v & 1) == 0; });
    ASSERT_TRUE((size_t)(mid - d.begin()) == evens);
    // a binary expression as the operator of reduce
    thrust::device_vector<long long> small(samples<long long>(1000, 10));
    long long sum_of = 0;
    thrust::host_vector<long long> hs = small;
    for (size_t i = 0; i < hs.size(); ++i) sum_of += hs[i];
    ASSERT_TRUE(thrust::reduce(small.begin(), small.end(), 0ll, _1 + _2) == sum_of);
  }
}

int main() {
  Arithmetic<int>();
  Arithmetic<unsigned int>();
  Arithmetic<float>();
  Arithmetic<long long>();
  Arithmetic<double>();
  IntegralOnly<int>();
  IntegralOnly<unsigned int>();
  IntegralOnly<short>();
  IntegralOnly<unsigned char>();
  LogicalAndRelational<int>();
  LogicalAndRelational<unsigned short>();
  LogicalAndRelational<float>();
  CompoundAssignment<int>();
  CompoundAssignment<float>();
  CompoundAssignment<long long>();
  CompoundAssignmentIntegral<int>();
  CompoundAssignmentIntegral<unsigned int>();
  CompoundAssignmentIntegral<short>();
  TestPlaceholdersInOtherAlgorithms();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
