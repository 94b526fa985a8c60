// Front-end test compiled with hipcc: the callers of reduce that answer "where" and "whether":
// min_element / max_element / minmax_element, find / find_if / find_if_not, all_of / any_of /
// none_of, mismatch, equal.  Literal vectors of the reference's unit tests
// (testing/min_element.cu:6-30, max_element.cu:6-30, minmax_element.cu:6-32, find.cu:44-132,
// logical.cu:8-122, mismatch.cu:6-40, equal.cu:6-50) on host_vector and device_vector, then the
// device system against the host system on random inputs of the reference's sizes.
#include <thrust/device_vector.h>
#include <thrust/equal.h>
#include <thrust/extrema.h>
#include <thrust/find.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/logical.h>
#include <thrust/mismatch.h>

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

static int g_failed = 0, g_checks = 0;
static const char* g_test = "";
#define ASSERT_TRUE(c)                                                                    \
  do {                                                                                    \
    ++g_checks;                                                                           \
    if (!(c)) { ++g_failed; std::printf("FAIL [%s] %s:%d: %s\n", g_test, __FILE__, __LINE__, #c); } \
  } while (0)
#define ASSERT_EQUAL(a, b) ASSERT_TRUE((a) == (b))

static uint64_t mix(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
template <typename T>
static thrust::host_vector<T> samples(size_t n, uint64_t seed, unsigned range) {
  thrust::host_vector<T> h(n);
  for (size_t i = 0; i < n; ++i) h[i] = (T)(mix(seed * 1000003ull + i) % range);
  return h;
}
static const size_t kSizes[] = {0, 1, 2, 3, 63, 64, 65, 1000, 4097, 100000, (1u << 20) + 7};

template <typename T>
struct equal_to_value_pred {
  T value;
  __host__ __device__ bool operator()(T v) const { return v == value; }
};
template <typename T>
struct not_equal_to_value_pred {
  T value;
  __host__ __device__ bool operator()(T v) const { return v != value; }
};
template <typename T>
struct less_than_value_pred {
  T value;
  __host__ __device__ bool operator()(T v) const { return v < value; }
};
struct by_last_digit {
  __host__ __device__ bool operator()(int a, int b) const { return a % 10 < b % 10; }
};

template <typename Vector>
static void Extrema() {
  typedef typename Vector::value_type T;
  g_test = "extrema: literal vectors";
  Vector data(6);
  data[0] = 3; data[1] = 5; data[2] = 1; data[3] = 2; data[4] = 5; data[5] = 1;
  ASSERT_EQUAL(*thrust::min_element(data.begin(), data.end()), T(1));
  ASSERT_EQUAL(thrust::min_element(data.begin(), data.end()) - data.begin(), 2);
  ASSERT_EQUAL(*thrust::min_element(data.begin(), data.end(), thrust::greater<T>()), T(5));
  ASSERT_EQUAL(thrust::min_element(data.begin(), data.end(), thrust::greater<T>()) - data.begin(), 1);
  ASSERT_EQUAL(*thrust::max_element(data.begin(), data.end()), T(5));
  ASSERT_EQUAL(thrust::max_element(data.begin(), data.end()) - data.begin(), 1);
  ASSERT_EQUAL(*thrust::max_element(data.begin(), data.end(), thrust::greater<T>()), T(1));
  ASSERT_EQUAL(thrust::max_element(data.begin(), data.end(), thrust::greater<T>()) - data.begin(), 2);
  ASSERT_EQUAL(*thrust::minmax_element(data.begin(), data.end()).first, T(1));
  ASSERT_EQUAL(*thrust::minmax_element(data.begin(), data.end()).second, T(5));
  ASSERT_EQUAL(thrust::minmax_element(data.begin(), data.end()).first - data.begin(), 2);
  ASSERT_EQUAL(thrust::minmax_element(data.begin(), data.end()).second - data.begin(), 1);
  // an empty range gives `last`
  ASSERT_TRUE(thrust::min_element(data.begin(), data.begin()) == data.begin());
  ASSERT_TRUE(thrust::max_element(data.begin(), data.begin()) == data.begin());
  ASSERT_TRUE(thrust::minmax_element(data.begin(), data.begin()).first == data.begin());
  ASSERT_TRUE(thrust::minmax_element(data.begin(), data.begin()).second == data.begin());
}

template <typename T>
static void ExtremaAgainstHost() {
  g_test = "extrema: device against host";
  for (size_t n : kSizes) {
    if (n == 0) continue;
    // few distinct values: many equivalent extremes, the first one must be named
    thrust::host_vector<T> h = samples<T>(n, 11 + n, n < 1000 ? 7 : 100);
    thrust::device_vector<T> d = h;
    ASSERT_EQUAL(thrust::min_element(d.begin(), d.end()) - d.begin(), thrust::min_element(h.begin(), h.end()) - h.begin());
    ASSERT_EQUAL(thrust::max_element(d.begin(), d.end()) - d.begin(), thrust::max_element(h.begin(), h.end()) - h.begin());
    ASSERT_EQUAL(thrust::min_element(d.begin(), d.end(), thrust::greater<T>()) - d.begin(),
                 thrust::min_element(h.begin(), h.end(), thrust::greater<T>()) - h.begin());
    ASSERT_EQUAL(thrust::minmax_element(d.begin(), d.end()).first - d.begin(),
                 thrust::minmax_element(h.begin(), h.end()).first - h.begin());
    ASSERT_EQUAL(thrust::minmax_element(d.begin(), d.end()).second - d.begin(),
                 thrust::minmax_element(h.begin(), h.end()).second - h.begin());
    // against the definition: no earlier element is as small, no element is smaller
    const size_t at = thrust::min_element(d.begin(), d.end()) - d.begin();
    bool first_smallest = true;
    for (size_t i = 0; i < n; ++i)
      if (h[i] < h[at] || (i < at && !(h[at] < h[i]))) first_smallest = false;
    ASSERT_TRUE(first_smallest);
  }
  // a comparison that makes different values equivalent
  thrust::host_vector<int> h = samples<int>(50000, 5, 1000);
  thrust::device_vector<int> d = h;
  ASSERT_EQUAL(thrust::min_element(d.begin(), d.end(), by_last_digit()) - d.begin(),
               thrust::min_element(h.begin(), h.end(), by_last_digit()) - h.begin());
  ASSERT_EQUAL(thrust::max_element(d.begin(), d.end(), by_last_digit()) - d.begin(),
               thrust::max_element(h.begin(), h.end(), by_last_digit()) - h.begin());
  // with an execution policy and raw pointers
  int* raw = thrust::raw_pointer_cast(d.data());
  ASSERT_EQUAL(thrust::min_element(thrust::device, raw, raw + d.size()) - raw,
               thrust::min_element(thrust::host, h.begin(), h.end()) - h.begin());
}

template <typename Vector>
static void Find() {
  typedef typename Vector::value_type T;
  g_test = "find: literal vectors";
  Vector vec(5);
  vec[0] = 1; vec[1] = 2; vec[2] = 3; vec[3] = 3; vec[4] = 5;
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 0) - vec.begin(), 5);
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 1) - vec.begin(), 0);
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 2) - vec.begin(), 1);
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 3) - vec.begin(), 2);
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 4) - vec.begin(), 5);
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 5) - vec.begin(), 4);
  for (int v = 0; v <= 5; ++v) {
    const int want[] = {5, 0, 1, 2, 5, 4};
    const equal_to_value_pred<T> is = {T(v)};
    ASSERT_EQUAL(thrust::find_if(vec.begin(), vec.end(), is) - vec.begin(), want[v]);
  }
  vec[0] = 0; vec[1] = 1; vec[2] = 2; vec[3] = 3; vec[4] = 4;
  for (int v = 0; v <= 5; ++v) {
    // the first element that is not below v
    const less_than_value_pred<T> below = {T(v)};
    ASSERT_EQUAL(thrust::find_if_not(vec.begin(), vec.end(), below) - vec.begin(), v);
  }
  const not_equal_to_value_pred<T> not_zero = {T(0)};
  ASSERT_EQUAL(thrust::find_if_not(vec.begin(), vec.end(), not_zero) - vec.begin(), 0);
}

template <typename T>
static void FindAgainstHost() {
  g_test = "find: device against host";
  for (size_t n : kSizes) {
    thrust::host_vector<T> h = samples<T>(n, 21 + n, 1000);
    thrust::device_vector<T> d = h;
    // present near the start, in the middle, at the end, absent
    const T probes[] = {n ? h[0] : T(1), n ? h[n / 2] : T(2), n ? h[n - 1] : T(3), T(5000)};
    for (T v : probes) {
      ASSERT_EQUAL(thrust::find(d.begin(), d.end(), v) - d.begin(), thrust::find(h.begin(), h.end(), v) - h.begin());
      const equal_to_value_pred<T> is = {v};
      ASSERT_EQUAL(thrust::find_if(d.begin(), d.end(), is) - d.begin(), thrust::find_if(h.begin(), h.end(), is) - h.begin());
      const not_equal_to_value_pred<T> is_not = {v};
      ASSERT_EQUAL(thrust::find_if_not(d.begin(), d.end(), is_not) - d.begin(),
                   thrust::find_if_not(h.begin(), h.end(), is_not) - h.begin());
    }
  }
}

template <typename Vector>
static void Logical() {
  typedef typename Vector::value_type T;
  g_test = "logical: literal vectors";
  Vector v(3, T(1));
  ASSERT_EQUAL(thrust::all_of(v.begin(), v.end(), thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::any_of(v.begin(), v.end(), thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::none_of(v.begin(), v.end(), thrust::identity<T>()), false);
  v[1] = 0;
  ASSERT_EQUAL(thrust::all_of(v.begin(), v.end(), thrust::identity<T>()), false);
  ASSERT_EQUAL(thrust::any_of(v.begin(), v.end(), thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::none_of(v.begin(), v.end(), thrust::identity<T>()), false);
  // empty and one-element ranges
  ASSERT_EQUAL(thrust::all_of(v.begin() + 0, v.begin() + 0, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::all_of(v.begin() + 0, v.begin() + 1, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::all_of(v.begin() + 0, v.begin() + 2, thrust::identity<T>()), false);
  ASSERT_EQUAL(thrust::all_of(v.begin() + 1, v.begin() + 2, thrust::identity<T>()), false);
  ASSERT_EQUAL(thrust::any_of(v.begin() + 0, v.begin() + 0, thrust::identity<T>()), false);
  ASSERT_EQUAL(thrust::any_of(v.begin() + 0, v.begin() + 1, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::any_of(v.begin() + 0, v.begin() + 2, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::any_of(v.begin() + 1, v.begin() + 2, thrust::identity<T>()), false);
  ASSERT_EQUAL(thrust::none_of(v.begin() + 0, v.begin() + 0, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::none_of(v.begin() + 0, v.begin() + 1, thrust::identity<T>()), false);
  ASSERT_EQUAL(thrust::none_of(v.begin() + 0, v.begin() + 2, thrust::identity<T>()), false);
  ASSERT_EQUAL(thrust::none_of(v.begin() + 1, v.begin() + 2, thrust::identity<T>()), true);
  // one failing element anywhere in a long range
  for (size_t at : {size_t(0), size_t(70001), size_t(199999)}) {
    Vector big(200000, T(1));
    ASSERT_EQUAL(thrust::all_of(big.begin(), big.end(), thrust::identity<T>()), true);
    big[at] = 0;
    ASSERT_EQUAL(thrust::all_of(big.begin(), big.end(), thrust::identity<T>()), false);
    ASSERT_EQUAL(thrust::any_of(big.begin(), big.end(), thrust::logical_not<T>()), true);
    ASSERT_EQUAL(thrust::none_of(big.begin(), big.end(), thrust::logical_not<T>()), false);
  }
}

template <typename Vector>
static void MismatchAndEqual() {
  typedef typename Vector::value_type T;
  g_test = "mismatch / equal: literal vectors";
  Vector a(4), b(4);
  a[0] = 1; a[1] = 2; a[2] = 3; a[3] = 4;
  b[0] = 1; b[1] = 2; b[2] = 4; b[3] = 3;
  ASSERT_EQUAL(thrust::mismatch(a.begin(), a.end(), b.begin()).first - a.begin(), 2);
  ASSERT_EQUAL(thrust::mismatch(a.begin(), a.end(), b.begin()).second - b.begin(), 2);
  b[2] = 3;
  ASSERT_EQUAL(thrust::mismatch(a.begin(), a.end(), b.begin()).first - a.begin(), 3);
  ASSERT_EQUAL(thrust::mismatch(a.begin(), a.end(), b.begin()).second - b.begin(), 3);
  b[3] = 4;
  ASSERT_EQUAL(thrust::mismatch(a.begin(), a.end(), b.begin()).first - a.begin(), 4);
  ASSERT_EQUAL(thrust::mismatch(a.begin(), a.end(), b.begin()).second - b.begin(), 4);
  // under a predicate: a[i] <= b[i] fails first where a exceeds b
  b[1] = 1;
  ASSERT_EQUAL(thrust::mismatch(a.begin(), a.end(), b.begin(), thrust::less_equal<T>()).first - a.begin(), 1);

  Vector v1(5), v2(5);
  v1[0] = 5; v1[1] = 2; v1[2] = 0; v1[3] = 0; v1[4] = 0;
  v2[0] = 5; v2[1] = 2; v2[2] = 0; v2[3] = 6; v2[4] = 1;
  ASSERT_EQUAL(thrust::equal(v1.begin(), v1.end(), v1.begin()), true);
  ASSERT_EQUAL(thrust::equal(v1.begin(), v1.end(), v2.begin()), false);
  ASSERT_EQUAL(thrust::equal(v2.begin(), v2.end(), v2.begin()), true);
  ASSERT_EQUAL(thrust::equal(v1.begin(), v1.begin() + 0, v1.begin()), true);
  ASSERT_EQUAL(thrust::equal(v1.begin(), v1.begin() + 1, v1.begin()), true);
  ASSERT_EQUAL(thrust::equal(v1.begin(), v1.begin() + 3, v2.begin()), true);
  ASSERT_EQUAL(thrust::equal(v1.begin(), v1.begin() + 4, v2.begin()), false);
  ASSERT_EQUAL(thrust::equal(v1.begin(), v1.end(), v2.begin(), thrust::less_equal<T>()), true);
  ASSERT_EQUAL(thrust::equal(v1.begin(), v1.end(), v2.begin(), thrust::greater<T>()), false);
}

template <typename T>
static void MismatchAgainstHost() {
  g_test = "mismatch / equal: device against host";
  for (size_t n : kSizes) {
    thrust::host_vector<T> h1 = samples<T>(n, 31 + n, 50), h2 = h1;
    thrust::device_vector<T> d1 = h1, d2 = h2;
    ASSERT_EQUAL(thrust::equal(d1.begin(), d1.end(), d2.begin()), true);
    ASSERT_EQUAL(thrust::mismatch(d1.begin(), d1.end(), d2.begin()).first - d1.begin(), (std::ptrdiff_t)n);
    if (n == 0) continue;
    for (size_t at : {size_t(0), n / 2, n - 1}) {
      h2 = h1;
      h2[at] = h2[at] + 1;
      if (at + 3 < n) h2[at + 3] = h2[at + 3] + 1;  // a later difference must not be reported
      d2 = h2;
      ASSERT_EQUAL(thrust::equal(d1.begin(), d1.end(), d2.begin()), false);
      ASSERT_EQUAL(thrust::mismatch(d1.begin(), d1.end(), d2.begin()).first - d1.begin(), (std::ptrdiff_t)at);
      ASSERT_EQUAL(thrust::mismatch(d1.begin(), d1.end(), d2.begin()).second - d2.begin(), (std::ptrdiff_t)at);
      ASSERT_EQUAL(thrust::mismatch(h1.begin(), h1.end(), h2.begin()).first - h1.begin(), (std::ptrdiff_t)at);
    }
  }
}

int main() {
  Extrema<thrust::host_vector<int> >();
  Extrema<thrust::device_vector<int> >();
  Extrema<thrust::device_vector<float> >();
  Extrema<thrust::device_vector<long long> >();
  Extrema<thrust::device_vector<signed char> >();
  ExtremaAgainstHost<int>();
  ExtremaAgainstHost<float>();
  ExtremaAgainstHost<unsigned long long>();
  ExtremaAgainstHost<short>();
  Find<thrust::host_vector<int> >();
  Find<thrust::device_vector<int> >();
  Find<thrust::device_vector<float> >();
  Find<thrust::device_vector<short> >();
  FindAgainstHost<int>();
  FindAgainstHost<double>();
  FindAgainstHost<unsigned short>();
  Logical<thrust::host_vector<int> >();
  Logical<thrust::device_vector<int> >();
  Logical<thrust::device_vector<unsigned char> >();
  MismatchAndEqual<thrust::host_vector<int> >();
  MismatchAndEqual<thrust::device_vector<int> >();
  MismatchAndEqual<thrust::device_vector<float> >();
  MismatchAgainstHost<int>();
  MismatchAgainstHost<long long>();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
