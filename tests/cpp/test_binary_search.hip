// Front-end test compiled with hipcc: lower_bound, upper_bound, binary_search, equal_range for one
// value and for ranges of values.  Literal vectors of the reference's unit tests
// (testing/binary_search.cu:50-170, binary_search_vector.cu:60-200, binary_search_descending.cu:6-120,
// binary_search_vector_descending.cu) on host_vector and device_vector, then the device system
// against the host system on sorted random inputs.
#include <thrust/binary_search.h>
#include <thrust/device_vector.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/sort.h>

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
template <typename A, typename B>
static bool same(const A& a, const B& b) {
  if (a.size() != b.size()) return false;
  for (size_t i = 0; i < a.size(); ++i)
    if (!(a[i] == b[i])) return false;
  return true;
}

struct by_tens {
  __host__ __device__ bool operator()(int a, int b) const { return a / 10 < b / 10; }
};

template <typename Vector>
static void Scalar() {
  typedef typename Vector::value_type T;
  g_test = "binary search, one value: literal vectors";
  Vector vec(5);
  vec[0] = 0; vec[1] = 2; vec[2] = 5; vec[3] = 7; vec[4] = 8;
  const int lower[] = {0, 1, 1, 2, 2, 2, 3, 3, 4, 5};
  const int upper[] = {1, 1, 2, 2, 2, 3, 3, 4, 5, 5};
  const bool found[] = {true, false, true, false, false, true, false, true, true, false};
  for (int v = 0; v < 10; ++v) {
    ASSERT_EQUAL(thrust::lower_bound(vec.begin(), vec.end(), T(v)) - vec.begin(), lower[v]);
    ASSERT_EQUAL(thrust::upper_bound(vec.begin(), vec.end(), T(v)) - vec.begin(), upper[v]);
    ASSERT_EQUAL(thrust::binary_search(vec.begin(), vec.end(), T(v)), found[v]);
    ASSERT_EQUAL(thrust::equal_range(vec.begin(), vec.end(), T(v)).first - vec.begin(), lower[v]);
    ASSERT_EQUAL(thrust::equal_range(vec.begin(), vec.end(), T(v)).second - vec.begin(), upper[v]);
    ASSERT_EQUAL(thrust::lower_bound(vec.begin(), vec.end(), T(v), thrust::less<T>()) - vec.begin(), lower[v]);
  }
  // descending, under greater
  vec[0] = 8; vec[1] = 7; vec[2] = 5; vec[3] = 2; vec[4] = 0;
  const int dlower[] = {4, 4, 3, 3, 3, 2, 2, 1, 0, 0};
  const int dupper[] = {5, 4, 4, 3, 3, 3, 2, 2, 1, 0};
  for (int v = 0; v < 10; ++v) {
    ASSERT_EQUAL(thrust::lower_bound(vec.begin(), vec.end(), T(v), thrust::greater<T>()) - vec.begin(), dlower[v]);
    ASSERT_EQUAL(thrust::upper_bound(vec.begin(), vec.end(), T(v), thrust::greater<T>()) - vec.begin(), dupper[v]);
    ASSERT_EQUAL(thrust::binary_search(vec.begin(), vec.end(), T(v), thrust::greater<T>()), found[v]);
  }
  // an empty range
  ASSERT_TRUE(thrust::lower_bound(vec.begin(), vec.begin(), T(3)) == vec.begin());
  ASSERT_TRUE(thrust::upper_bound(vec.begin(), vec.begin(), T(3)) == vec.begin());
  ASSERT_EQUAL(thrust::binary_search(vec.begin(), vec.begin(), T(3)), false);
}

template <typename Vector, typename IntVector>
static void Vectorised() {
  typedef typename Vector::value_type T;
  g_test = "binary search, ranges of values: literal vectors";
  Vector vec(5);
  vec[0] = 0; vec[1] = 2; vec[2] = 5; vec[3] = 7; vec[4] = 8;
  Vector input(10);
  for (int v = 0; v < 10; ++v) input[v] = T(v);
  IntVector out(10);
  const int lower[] = {0, 1, 1, 2, 2, 2, 3, 3, 4, 5};
  const int upper[] = {1, 1, 2, 2, 2, 3, 3, 4, 5, 5};
  const int found[] = {1, 0, 1, 0, 0, 1, 0, 1, 1, 0};
  auto end = thrust::lower_bound(vec.begin(), vec.end(), input.begin(), input.end(), out.begin());
  ASSERT_EQUAL(end - out.begin(), 10);
  for (int v = 0; v < 10; ++v) ASSERT_EQUAL((int)out[v], lower[v]);
  end = thrust::upper_bound(vec.begin(), vec.end(), input.begin(), input.end(), out.begin());
  ASSERT_EQUAL(end - out.begin(), 10);
  for (int v = 0; v < 10; ++v) ASSERT_EQUAL((int)out[v], upper[v]);
  end = thrust::binary_search(vec.begin(), vec.end(), input.begin(), input.end(), out.begin());
  ASSERT_EQUAL(end - out.begin(), 10);
  for (int v = 0; v < 10; ++v) ASSERT_EQUAL((int)out[v], found[v]);
  // descending
  vec[0] = 8; vec[1] = 7; vec[2] = 5; vec[3] = 2; vec[4] = 0;
  const int dlower[] = {4, 4, 3, 3, 3, 2, 2, 1, 0, 0};
  const int dupper[] = {5, 4, 4, 3, 3, 3, 2, 2, 1, 0};
  thrust::lower_bound(vec.begin(), vec.end(), input.begin(), input.end(), out.begin(), thrust::greater<T>());
  for (int v = 0; v < 10; ++v) ASSERT_EQUAL((int)out[v], dlower[v]);
  thrust::upper_bound(vec.begin(), vec.end(), input.begin(), input.end(), out.begin(), thrust::greater<T>());
  for (int v = 0; v < 10; ++v) ASSERT_EQUAL((int)out[v], dupper[v]);
  thrust::binary_search(vec.begin(), vec.end(), input.begin(), input.end(), out.begin(), thrust::greater<T>());
  for (int v = 0; v < 10; ++v) ASSERT_EQUAL((int)out[v], found[v]);
}

template <typename T>
static void AgainstHost() {
  g_test = "binary search: device against host";
  const size_t sizes[] = {0, 1, 2, 63, 1000, 4097, 100000, (1u << 20) + 7};
  for (size_t n : sizes) {
    thrust::host_vector<T> h = samples<T>(n, 81 + n, n < 1000 ? 20 : 5000);
    thrust::sort(h.begin(), h.end());
    thrust::device_vector<T> d = h;
    const size_t m = n < 1000 ? 100 : 20000;
    thrust::host_vector<T> hv = samples<T>(m, 82 + n, n < 1000 ? 25 : 5200);  // some beyond the largest element
    thrust::device_vector<T> dv = hv;
    thrust::host_vector<long long> ho(m);
    thrust::device_vector<long long> dout(m);
    thrust::lower_bound(h.begin(), h.end(), hv.begin(), hv.end(), ho.begin());
    thrust::lower_bound(d.begin(), d.end(), dv.begin(), dv.end(), dout.begin());
    ASSERT_TRUE(same(thrust::host_vector<long long>(dout), ho));
    thrust::upper_bound(h.begin(), h.end(), hv.begin(), hv.end(), ho.begin());
    thrust::upper_bound(d.begin(), d.end(), dv.begin(), dv.end(), dout.begin());
    ASSERT_TRUE(same(thrust::host_vector<long long>(dout), ho));
    thrust::host_vector<bool> hb(m);
    thrust::device_vector<bool> db(m);
    thrust::binary_search(h.begin(), h.end(), hv.begin(), hv.end(), hb.begin());
    thrust::binary_search(d.begin(), d.end(), dv.begin(), dv.end(), db.begin());
    ASSERT_TRUE(same(thrust::host_vector<bool>(db), hb));
    for (size_t i = 0; i < 5 && i < m; ++i) {
      ASSERT_EQUAL(thrust::lower_bound(d.begin(), d.end(), hv[i]) - d.begin(), thrust::lower_bound(h.begin(), h.end(), hv[i]) - h.begin());
      ASSERT_EQUAL(thrust::upper_bound(d.begin(), d.end(), hv[i]) - d.begin(), thrust::upper_bound(h.begin(), h.end(), hv[i]) - h.begin());
      ASSERT_EQUAL(thrust::binary_search(d.begin(), d.end(), hv[i]), thrust::binary_search(h.begin(), h.end(), hv[i]));
    }
  }
  // a comparison that makes different values equivalent: the bounds enclose the whole class
  thrust::host_vector<int> h = samples<int>(30000, 9, 2000);
  thrust::sort(h.begin(), h.end());
  thrust::device_vector<int> d = h;
  for (int v : {0, 15, 999, 1995, 2500}) {
    ASSERT_EQUAL(thrust::lower_bound(d.begin(), d.end(), v, by_tens()) - d.begin(), thrust::lower_bound(h.begin(), h.end(), v, by_tens()) - h.begin());
    ASSERT_EQUAL(thrust::upper_bound(d.begin(), d.end(), v, by_tens()) - d.begin(), thrust::upper_bound(h.begin(), h.end(), v, by_tens()) - h.begin());
    ASSERT_EQUAL(thrust::equal_range(d.begin(), d.end(), v, by_tens()).second - d.begin(),
                 thrust::equal_range(h.begin(), h.end(), v, by_tens()).second - h.begin());
  }
}

int main() {
  Scalar<thrust::host_vector<int> >();
  Scalar<thrust::device_vector<int> >();
  Scalar<thrust::device_vector<float> >();
  Scalar<thrust::device_vector<short> >();
  Vectorised<thrust::host_vector<int>, thrust::host_vector<int> >();
  Vectorised<thrust::device_vector<int>, thrust::device_vector<int> >();
  Vectorised<thrust::device_vector<double>, thrust::device_vector<int> >();
  AgainstHost<int>();
  AgainstHost<unsigned int>();
  AgainstHost<float>();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
