// Front-end tests: the unchanged thrust:: API on the gfx950 device system.
//
// Part 1 replays the literal known-answer vectors of the reference's own unit tests
// (cited per test) on device_vector.  Part 2 is the reference's differential pattern:
// the same algorithm on host_vector (sequential host system) and device_vector over the
// reference's size list, results compared exactly (testing/unittest/testframework.cu:21-31,
// e.g. testing/reduce.cu:80-95).  Part 3 covers policies, streams, dispatch interception,
// the memory model and error reporting.
#include <map>
#include <stdexcept>

#include <thrust/async/copy.h>
#include <thrust/async/reduce.h>
#include <thrust/async/scan.h>
#include <thrust/async/sort.h>
#include <thrust/copy.h>
#include <thrust/count.h>
#include <thrust/device_allocator.h>
#include <thrust/device_vector.h>
#include <thrust/execution_policy.h>
#include <thrust/fill.h>
#include <thrust/functional.h>
#include <thrust/future.h>
#include <thrust/host_vector.h>
#include <thrust/inner_product.h>
#include <thrust/merge.h>
#include <thrust/mr/allocator.h>
#include <thrust/mr/disjoint_pool.h>
#include <thrust/mr/disjoint_sync_pool.h>
#include <thrust/mr/new.h>
#include <thrust/mr/pool.h>
#include <thrust/mr/sync_pool.h>
#include <thrust/partition.h>
#include <thrust/reduce.h>
#include <thrust/remove.h>
#include <thrust/scan.h>
#include <thrust/set_operations.h>
#include <thrust/sort.h>
#include <thrust/transform_reduce.h>
#include <thrust/transform_scan.h>
#include <thrust/unique.h>
#include <thrust/universal_vector.h>

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <functional>
#include <limits>
#include <string>
#include <thread>
#include <vector>

static int g_failed = 0, g_checks = 0;
static const char* g_test = "";

#define ASSERT_TRUE(c)                                                                    \
  do {                                                                                    \
    ++g_checks;                                                                           \
    if (!(c)) { ++g_failed; std::printf("FAIL [%s] %s:%d: %s\n", g_test, __FILE__, __LINE__, #c); } \
  } while (0)

template <typename A, typename B>
static bool same(const A& a, const B& b) {
  if (a.size() != b.size()) return false;
  for (size_t i = 0; i < a.size(); ++i)
    if (!(a[i] == b[i])) return false;
  return true;
}
#define ASSERT_EQUAL_VEC(a, b) ASSERT_TRUE(same((a), (b)))

template <typename T>
static thrust::host_vector<T> hv(std::initializer_list<T> l) { return thrust::host_vector<T>(std::vector<T>(l)); }
template <typename T, typename A>
static thrust::host_vector<T> to_host(const thrust::device_vector<T, A>& d) { return thrust::host_vector<T>(d); }
template <typename T>
static thrust::host_vector<T> to_host(const thrust::host_vector<T>& h) { return h; }

// deterministic inputs: an index hash, in the spirit of testing/unittest/random.h:12-21
static uint64_t mix(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
template <typename T>
static thrust::host_vector<T> random_integers(size_t n, uint64_t seed, uint64_t modulus = 0) {
  thrust::host_vector<T> h(n);
  for (size_t i = 0; i < n; ++i) {
    const uint64_t r = mix(seed * 1000003ull + i);
    h[i] = (T)(modulus ? (r % modulus) : r);
  }
  return h;
}

static const size_t kSizes[] = {0, 1, 2, 3, 4, 5, 8, 10, 13, 16, 17, 19, 27, 30, 31, 32, 33, 35, 42, 53, 58, 63,
                                64, 65, 72, 97, 100, 127, 128, 129, 142, 183, 192, 201, 240, 255, 256, 257, 302,
                                511, 512, 513, 687, 900, 1023, 1024, 1025, 1565, 1786, 1973, 2047, 2048, 2049,
                                3050, 4095, 4096, 4097, 5030, 7791, 10000, 10027, 12345, 16384, 17354, 26255,
                                32768, 43718, 65533, 65536, 65539};

using namespace thrust::placeholders;

// ================================================================ part 1: known answers
static void TestReduceSimple() {  // testing/reduce.cu:26-39
  g_test = "ReduceSimple";
  thrust::device_vector<int> v(hv<int>({1, -2, 3}));
  ASSERT_TRUE(thrust::reduce(v.begin(), v.end()) == 2);
  ASSERT_TRUE(thrust::reduce(v.begin(), v.end(), 10) == 12);
  ASSERT_TRUE(thrust::reduce(v.begin(), v.end(), 10, thrust::plus<int>()) == 12);
  ASSERT_TRUE(thrust::reduce(thrust::device, v.begin(), v.end(), 10) == 12);
  ASSERT_TRUE(thrust::reduce(v.begin(), v.end(), 0, thrust::maximum<int>()) == 3);
  ASSERT_TRUE(thrust::reduce(v.begin(), v.end(), 0, thrust::minimum<int>()) == -2);
  ASSERT_TRUE(thrust::reduce(v.begin(), v.begin(), 7) == 7);  // empty range returns init
}

static void TestReduceWithOperatorTable() {  // the data of testing/reduce.cu:166-192, plain plus here
  g_test = "ReduceTable";
  thrust::device_vector<unsigned int> v(hv<unsigned int>({0, 1, 2, 1, 2, 0, 1}));
  ASSERT_TRUE(thrust::reduce(v.begin(), v.end()) == 7u);
}

static void TestScanSimple() {  // testing/scan.cu:23-93
  g_test = "ScanSimple";
  const thrust::host_vector<int> in = hv<int>({1, 3, -2, 4, -5});
  thrust::device_vector<int> input(in), output(5, 0);
  auto it = thrust::inclusive_scan(input.begin(), input.end(), output.begin());
  ASSERT_TRUE(it - output.begin() == 5);
  ASSERT_EQUAL_VEC(to_host(input), in);
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({1, 4, 2, 6, 1}));
  it = thrust::exclusive_scan(input.begin(), input.end(), output.begin(), 0);
  ASSERT_TRUE(it - output.begin() == 5);
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({0, 1, 4, 2, 6}));
  thrust::exclusive_scan(input.begin(), input.end(), output.begin(), 3);
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({3, 4, 7, 5, 9}));
  // inclusive scan with op
  thrust::inclusive_scan(input.begin(), input.end(), output.begin(), thrust::plus<int>());
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({1, 4, 2, 6, 1}));
  // exclusive scan with init and op
  thrust::exclusive_scan(input.begin(), input.end(), output.begin(), 3, thrust::plus<int>());
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({3, 4, 7, 5, 9}));
  // in-place
  input = in;
  thrust::inclusive_scan(input.begin(), input.end(), input.begin(), thrust::plus<int>());
  ASSERT_EQUAL_VEC(to_host(input), hv<int>({1, 4, 2, 6, 1}));
  input = in;
  thrust::exclusive_scan(input.begin(), input.end(), input.begin(), 3, thrust::plus<int>());
  ASSERT_EQUAL_VEC(to_host(input), hv<int>({3, 4, 7, 5, 9}));
  // exclusive_scan without init starts from 0
  input = in;
  thrust::exclusive_scan(input.begin(), input.end(), output.begin());
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({0, 1, 4, 2, 6}));
}

// testing/reduce.cu:98-129 and testing/scan.cu:236-295: the accumulator is init's type for
// reduce and exclusive_scan and the input's type for inclusive_scan; the plus<int>-on-float
// case of the scan test is outside the device system's operator set and is left out.
template <typename IntVector, typename FloatVector>
static void MixedTypes() {
  IntVector int_input(hv<int>({1, 2, 3, 4}));
  FloatVector float_input(hv<float>({1.5f, 2.5f, 3.5f, 4.5f}));
  ASSERT_TRUE(thrust::reduce(float_input.begin(), float_input.end(), (int)0) == 10);
  ASSERT_TRUE(thrust::reduce(int_input.begin(), int_input.end(), (float)0.5) == 10.5f);

  IntVector int_output(4);
  FloatVector float_output(4);
  thrust::inclusive_scan(float_input.begin(), float_input.end(), int_output.begin());
  ASSERT_EQUAL_VEC(to_host(int_output), hv<int>({1, 4, 7, 12}));
  thrust::exclusive_scan(float_input.begin(), float_input.end(), int_output.begin());
  ASSERT_EQUAL_VEC(to_host(int_output), hv<int>({0, 1, 4, 7}));
  thrust::exclusive_scan(float_input.begin(), float_input.end(), int_output.begin(), (float)5.5);
  ASSERT_EQUAL_VEC(to_host(int_output), hv<int>({5, 7, 9, 13}));
  thrust::inclusive_scan(int_input.begin(), int_input.end(), float_output.begin());
  ASSERT_EQUAL_VEC(to_host(float_output), hv<float>({1.f, 3.f, 6.f, 10.f}));
  thrust::exclusive_scan(int_input.begin(), int_input.end(), float_output.begin(), (float)5.5);
  ASSERT_EQUAL_VEC(to_host(float_output), hv<float>({5.5f, 6.5f, 8.5f, 11.5f}));
}

static void TestMixedTypes() {
  g_test = "MixedTypesHost";
  MixedTypes<thrust::host_vector<int>, thrust::host_vector<float>>();
  g_test = "MixedTypesDevice";
  MixedTypes<thrust::device_vector<int>, thrust::device_vector<float>>();

  // widening and narrowing at a size that spans several tiles, against the host system
  g_test = "MixedTypesLarge";
  const std::size_t n = 100003;
  thrust::host_vector<short> h(n);
  for (std::size_t i = 0; i < n; ++i) h[i] = (short)((i * 2654435761u >> 7) % 2001) - 1000;
  thrust::device_vector<short> d(h);
  ASSERT_TRUE(thrust::reduce(d.begin(), d.end(), (long long)5) == thrust::reduce(h.begin(), h.end(), (long long)5));
  ASSERT_TRUE(thrust::reduce(d.begin(), d.end(), (long long)-7, thrust::maximum<long long>()) ==
              thrust::reduce(h.begin(), h.end(), (long long)-7, thrust::maximum<long long>()));
  thrust::host_vector<long long> h_wide(n);
  thrust::device_vector<long long> d_wide(n);
  thrust::exclusive_scan(h.begin(), h.end(), h_wide.begin(), (long long)1 << 40);
  thrust::exclusive_scan(d.begin(), d.end(), d_wide.begin(), (long long)1 << 40);
  ASSERT_EQUAL_VEC(to_host(d_wide), h_wide);
  thrust::inclusive_scan(h.begin(), h.end(), h_wide.begin());  // short accumulator wraps, then widens
  thrust::inclusive_scan(d.begin(), d.end(), d_wide.begin());
  ASSERT_EQUAL_VEC(to_host(d_wide), h_wide);
  thrust::host_vector<unsigned char> h_narrow(n);
  thrust::device_vector<unsigned char> d_narrow(n);
  thrust::exclusive_scan(h.begin(), h.end(), h_narrow.begin(), 3);  // int accumulator, bytes out
  thrust::exclusive_scan(d.begin(), d.end(), d_narrow.begin(), 3);
  ASSERT_EQUAL_VEC(to_host(d_narrow), h_narrow);
}

static void TestScanByKeySimple() {  // testing/scan_by_key.cu:9-60 and :121-180
  g_test = "ScanByKeySimple";
  thrust::device_vector<int> keys(hv<int>({0, 1, 1, 1, 2, 3, 3})), vals(hv<int>({1, 2, 3, 4, 5, 6, 7})), output(7, 0);
  auto it = thrust::inclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin());
  ASSERT_TRUE(it - output.begin() == 7);
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({1, 2, 5, 9, 5, 6, 13}));
  thrust::inclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin(), thrust::equal_to<int>());
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({1, 2, 5, 9, 5, 6, 13}));
  thrust::inclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin(), thrust::equal_to<int>(),
                                thrust::maximum<int>());
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({1, 2, 3, 4, 5, 6, 7}));
  it = thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin());
  ASSERT_TRUE(it - output.begin() == 7);
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({0, 0, 2, 5, 0, 0, 6}));
  thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin(), 10);
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({10, 10, 12, 15, 10, 10, 16}));
  thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin(), 10, thrust::equal_to<int>());
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({10, 10, 12, 15, 10, 10, 16}));
  thrust::exclusive_scan_by_key(thrust::device, keys.begin(), keys.end(), vals.begin(), output.begin(), 10,
                                thrust::equal_to<int>(), thrust::plus<int>());
  ASSERT_EQUAL_VEC(to_host(output), hv<int>({10, 10, 12, 15, 10, 10, 16}));
  // in place, both forms
  thrust::device_vector<int> v2 = vals;
  thrust::inclusive_scan_by_key(keys.begin(), keys.end(), v2.begin(), v2.begin());
  ASSERT_EQUAL_VEC(to_host(v2), hv<int>({1, 2, 5, 9, 5, 6, 13}));
  v2 = vals;
  thrust::exclusive_scan_by_key(keys.begin(), keys.end(), v2.begin(), v2.begin(), 10);
  ASSERT_EQUAL_VEC(to_host(v2), hv<int>({10, 10, 12, 15, 10, 10, 16}));
  // the host system gives the same answers
  thrust::host_vector<int> hk = to_host(keys), hvals = to_host(vals), ho(7);
  thrust::inclusive_scan_by_key(hk.begin(), hk.end(), hvals.begin(), ho.begin());
  ASSERT_EQUAL_VEC(ho, hv<int>({1, 2, 5, 9, 5, 6, 13}));
  thrust::exclusive_scan_by_key(hk.begin(), hk.end(), hvals.begin(), ho.begin(), 10);
  ASSERT_EQUAL_VEC(ho, hv<int>({10, 10, 12, 15, 10, 10, 16}));
}

static void TestCountSimple() {  // testing/count.cu:5-14 and :40-49
  g_test = "CountSimple";
  thrust::device_vector<int> data(hv<int>({1, 1, 0, 0, 1}));
  ASSERT_TRUE(thrust::count(data.begin(), data.end(), 0) == 2);
  ASSERT_TRUE(thrust::count(data.begin(), data.end(), 1) == 3);
  ASSERT_TRUE(thrust::count(data.begin(), data.end(), 2) == 0);
  thrust::device_vector<int> d2(hv<int>({1, 6, 1, 9, 2}));
  ASSERT_TRUE(thrust::count_if(d2.begin(), d2.end(), _1 > 5) == 2);
  ASSERT_TRUE(thrust::count_if(thrust::device, d2.begin(), d2.end(), _1 > 5) == 2);
  thrust::host_vector<int> h2 = to_host(d2);
  ASSERT_TRUE(thrust::count_if(h2.begin(), h2.end(), _1 > 5) == 2);
  ASSERT_TRUE(thrust::count(h2.begin(), h2.end(), 1) == 2);
}

static void TestInnerProductSimple() {  // testing/inner_product.cu:10-24
  g_test = "InnerProductSimple";
  thrust::device_vector<int> v1(hv<int>({1, -2, 3})), v2(hv<int>({-4, 5, 6}));
  ASSERT_TRUE(thrust::inner_product(v1.begin(), v1.end(), v2.begin(), 3) == 7);
  ASSERT_TRUE(thrust::inner_product(thrust::device, v1.begin(), v1.end(), v2.begin(), 3) == 7);
  ASSERT_TRUE(thrust::inner_product(v1.begin(), v1.end(), v2.begin(), 3, thrust::plus<int>(), thrust::multiplies<int>()) == 7);
  thrust::host_vector<int> h1 = to_host(v1), h2 = to_host(v2);
  ASSERT_TRUE(thrust::inner_product(h1.begin(), h1.end(), h2.begin(), 3) == 7);
}

static void TestTransformReduceAndScanSimple() {  // testing/transform_reduce.cu:70-83, transform_scan.cu:140-190,355-399
  g_test = "TransformReduceAndScanSimple";
  thrust::device_vector<int> data(hv<int>({1, -2, 3}));
  ASSERT_TRUE(thrust::transform_reduce(data.begin(), data.end(), thrust::negate<int>(), 10, thrust::plus<int>()) == 8);
  ASSERT_TRUE(thrust::transform_reduce(thrust::device, data.begin(), data.end(), thrust::square<int>(), 1, thrust::plus<int>()) == 15);
  thrust::host_vector<int> hdata = to_host(data);
  ASSERT_TRUE(thrust::transform_reduce(hdata.begin(), hdata.end(), thrust::negate<int>(), 10, thrust::plus<int>()) == 8);
  thrust::device_vector<int> in(hv<int>({1, 3, -2, 4, -5})), out(5);
  auto it = thrust::transform_inclusive_scan(in.begin(), in.end(), out.begin(), thrust::negate<int>(), thrust::plus<int>());
  ASSERT_TRUE(it - out.begin() == 5);
  ASSERT_EQUAL_VEC(to_host(out), hv<int>({-1, -4, -2, -6, -1}));
  ASSERT_EQUAL_VEC(to_host(in), hv<int>({1, 3, -2, 4, -5}));
  thrust::transform_exclusive_scan(in.begin(), in.end(), out.begin(), thrust::negate<int>(), 0, thrust::plus<int>());
  ASSERT_EQUAL_VEC(to_host(out), hv<int>({0, -1, -4, -2, -6}));
  thrust::transform_exclusive_scan(thrust::device, in.begin(), in.end(), out.begin(), thrust::negate<int>(), 3, thrust::plus<int>());
  ASSERT_EQUAL_VEC(to_host(out), hv<int>({3, 2, -1, 1, -3}));
  thrust::device_vector<int> inplace = in;  // in place
  thrust::transform_inclusive_scan(inplace.begin(), inplace.end(), inplace.begin(), thrust::negate<int>(), thrust::plus<int>());
  ASSERT_EQUAL_VEC(to_host(inplace), hv<int>({-1, -4, -2, -6, -1}));
  inplace = in;
  thrust::transform_exclusive_scan(inplace.begin(), inplace.end(), inplace.begin(), thrust::negate<int>(), 3, thrust::plus<int>());
  ASSERT_EQUAL_VEC(to_host(inplace), hv<int>({3, 2, -1, 1, -3}));
  thrust::host_vector<int> hin = to_host(in), hout(5);
  thrust::transform_inclusive_scan(hin.begin(), hin.end(), hout.begin(), thrust::negate<int>(), thrust::plus<int>());
  ASSERT_EQUAL_VEC(hout, hv<int>({-1, -4, -2, -6, -1}));
  thrust::device_vector<int> vec(hv<int>({5, 0, 5, 8, 6, 7, 5, 3, 0, 9}));
  thrust::transform_inclusive_scan(thrust::device, vec.cbegin(), vec.cend(), vec.begin(), thrust::identity<>{}, thrust::maximum<>{});
  ASSERT_EQUAL_VEC(to_host(vec), hv<int>({5, 5, 5, 8, 8, 8, 8, 8, 8, 9}));
  vec = thrust::device_vector<int>(hv<int>({5, 0, 5, 8, 6, 7, 5, 3, 0, 9}));
  thrust::transform_exclusive_scan(thrust::device, vec.cbegin(), vec.cend(), vec.begin(), thrust::identity<>{}, int{}, thrust::maximum<>{});
  ASSERT_EQUAL_VEC(to_host(vec), hv<int>({0, 5, 5, 5, 8, 8, 8, 8, 8, 8}));
}

static void TestRemoveSimple() {  // testing/remove.cu:28-47,100-122,184-203,256-283,345-367,429-460
  g_test = "RemoveSimple";
  const thrust::host_vector<int> src = hv<int>({1, 2, 1, 3, 2});
  const thrust::host_vector<int> kept = hv<int>({1, 1, 3});
  thrust::device_vector<int> data(src);
  auto end = thrust::remove(data.begin(), data.end(), 2);
  ASSERT_TRUE(end - data.begin() == 3);
  data.resize(3);
  ASSERT_EQUAL_VEC(to_host(data), kept);
  data = thrust::device_vector<int>(src);
  thrust::device_vector<int> result(5);
  auto rend = thrust::remove_copy(data.begin(), data.end(), result.begin(), 2);
  ASSERT_TRUE(rend - result.begin() == 3);
  result.resize(3);
  ASSERT_EQUAL_VEC(to_host(result), kept);
  ASSERT_EQUAL_VEC(to_host(data), src);
  end = thrust::remove_if(data.begin(), data.end(), _1 == 2);
  ASSERT_TRUE(end - data.begin() == 3);
  data.resize(3);
  ASSERT_EQUAL_VEC(to_host(data), kept);
  data = thrust::device_vector<int>(src);
  thrust::device_vector<int> stencil(hv<int>({0, 1, 0, 0, 1}));
  end = thrust::remove_if(thrust::device, data.begin(), data.end(), stencil.begin(), thrust::identity<int>());
  ASSERT_TRUE(end - data.begin() == 3);
  data.resize(3);
  ASSERT_EQUAL_VEC(to_host(data), kept);
  data = thrust::device_vector<int>(src);
  result = thrust::device_vector<int>(5);
  rend = thrust::remove_copy_if(data.begin(), data.end(), result.begin(), _1 == 2);
  ASSERT_TRUE(rend - result.begin() == 3);
  rend = thrust::remove_copy_if(data.begin(), data.end(), stencil.begin(), result.begin(), thrust::identity<int>());
  ASSERT_TRUE(rend - result.begin() == 3);
  result.resize(3);
  ASSERT_EQUAL_VEC(to_host(result), kept);
  thrust::host_vector<int> h = src;  // the host system
  h.resize(thrust::remove(h.begin(), h.end(), 2) - h.begin());
  ASSERT_EQUAL_VEC(h, kept);
  h = src;
  thrust::host_vector<int> hst = hv<int>({0, 1, 0, 0, 1});
  h.resize(thrust::remove_if(h.begin(), h.end(), hst.begin(), thrust::identity<int>()) - h.begin());
  ASSERT_EQUAL_VEC(h, kept);
}

// Placeholder thresholds of another type than the elements: the device must select what C++
// selects under the usual arithmetic conversions (the host system evaluates the expression
// as written).  Covers a fractional threshold on integers, thresholds outside the element
// type's range, a negative threshold on unsigned elements and an integer threshold on floats.
template <typename T, typename Pred>
static void check_mixed_predicate(const thrust::host_vector<T>& h, Pred pred) {
  thrust::device_vector<T> d = h;
  thrust::host_vector<T> want(h.size());
  want.resize(thrust::copy_if(h.begin(), h.end(), want.begin(), pred) - want.begin());
  thrust::device_vector<T> got(h.size());
  got.resize(thrust::copy_if(d.begin(), d.end(), got.begin(), pred) - got.begin());
  ASSERT_EQUAL_VEC(to_host(got), want);
  ASSERT_TRUE((size_t)thrust::count_if(d.begin(), d.end(), pred) == want.size());
  thrust::host_vector<T> hr = h;
  hr.resize(thrust::remove_if(hr.begin(), hr.end(), pred) - hr.begin());
  thrust::device_vector<T> dr = h;
  dr.resize(thrust::remove_if(dr.begin(), dr.end(), pred) - dr.begin());
  ASSERT_EQUAL_VEC(to_host(dr), hr);
}
static void TestMixedTypePlaceholders() {
  g_test = "MixedTypePlaceholders";
  using namespace thrust::placeholders;
  const size_t n = 4099;
  {
    thrust::host_vector<int> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = (int)(mix(i) % 11) - 5;
    check_mixed_predicate(h, _1 < 2.5);
    check_mixed_predicate(h, _1 <= 2.5);
    check_mixed_predicate(h, _1 > -2.5);
    check_mixed_predicate(h, _1 >= -0.5);
    check_mixed_predicate(h, _1 == 2.5);
    check_mixed_predicate(h, _1 != 2.5);
    check_mixed_predicate(h, _1 == 2.0);
    check_mixed_predicate(h, _1 < 1e30);
    check_mixed_predicate(h, _1 > 1e30);
    check_mixed_predicate(h, _1 < 3ll);
    check_mixed_predicate(h, _1 < (1ll << 40));
    check_mixed_predicate(h, _1 >= -(1ll << 40));
    check_mixed_predicate(h, _1 != (1ll << 40));
  }
  {
    thrust::host_vector<int8_t> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = (int8_t)(mix(i) & 0xff);
    check_mixed_predicate(h, _1 > 300);   // wraps to 44 if the threshold is cast to int8
    check_mixed_predicate(h, _1 < 300);
    check_mixed_predicate(h, _1 == 300);
    check_mixed_predicate(h, _1 >= -200);
    check_mixed_predicate(h, _1 < 17);
    check_mixed_predicate(h, _1 < 16.5);
  }
  {
    thrust::host_vector<uint16_t> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = (uint16_t)(mix(i) & 0xffff);
    check_mixed_predicate(h, _1 > -1);     // compared as int: always true
    check_mixed_predicate(h, _1 < 70000);
    check_mixed_predicate(h, _1 >= 32768);
  }
  {
    thrust::host_vector<uint32_t> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = (uint32_t)mix(i);
    check_mixed_predicate(h, _1 < -2);     // compared as unsigned: below 4294967294
    check_mixed_predicate(h, _1 > 1000);
    check_mixed_predicate(h, _1 < (1ll << 31));
  }
  {
    thrust::host_vector<float> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = (float)((double)(mix(i) % 2001) / 250.0 - 4.0);
    check_mixed_predicate(h, _1 < 2);      // 2.5f < 2 is false: compared as float, not as int
    check_mixed_predicate(h, _1 == 2);
    check_mixed_predicate(h, _1 >= -1);
  }
  {
    thrust::host_vector<double> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = (double)(mix(i) % 2001) / 250.0 - 4.0;
    check_mixed_predicate(h, _1 < 0.3f);
    check_mixed_predicate(h, _1 > 1);
  }
}

// remove_if keeps what the predicate rejects.  A NaN fails `x < t` and is kept; it also fails
// `x >= t`, so the complementary comparison would drop it.
static void TestRemoveIfKeepsNaN() {
  g_test = "RemoveIfKeepsNaN";
  using namespace thrust::placeholders;
  const size_t n = 5000;
  const float nan = std::numeric_limits<float>::quiet_NaN();
  thrust::host_vector<float> h(n);
  size_t nans = 0;
  for (size_t i = 0; i < n; ++i) {
    h[i] = (mix(i) % 7 == 0) ? nan : (float)(mix(i) % 1000) / 1000.0f;
    nans += h[i] != h[i];
  }
  auto bits = [](const thrust::host_vector<float>& v) {
    thrust::host_vector<uint32_t> b(v.size());
    for (size_t i = 0; i < v.size(); ++i) std::memcpy(&b[i], &v[i], 4);
    return b;
  };
  thrust::host_vector<float> hr = h;
  hr.resize(thrust::remove_if(hr.begin(), hr.end(), _1 < 0.5f) - hr.begin());
  thrust::device_vector<float> dr = h;
  dr.resize(thrust::remove_if(dr.begin(), dr.end(), _1 < 0.5f) - dr.begin());
  ASSERT_EQUAL_VEC(bits(to_host(dr)), bits(hr));
  size_t kept_nans = 0;
  thrust::host_vector<float> back = dr;
  for (size_t i = 0; i < back.size(); ++i) kept_nans += back[i] != back[i];
  ASSERT_TRUE(kept_nans == nans && nans > 0);
  thrust::device_vector<float> d = h, out(n);
  out.resize(thrust::remove_copy_if(d.begin(), d.end(), out.begin(), _1 >= 0.5f) - out.begin());
  thrust::host_vector<float> hout(n);
  hout.resize(thrust::remove_copy_if(h.begin(), h.end(), hout.begin(), _1 >= 0.5f) - hout.begin());
  ASSERT_EQUAL_VEC(bits(to_host(out)), bits(hout));
  // partition: the NaNs fail the predicate and go behind the split point, in order
  thrust::host_vector<float> hp = h;
  thrust::device_vector<float> dp = h;
  const size_t hs = thrust::stable_partition(hp.begin(), hp.end(), _1 < 0.5f) - hp.begin();
  const size_t ds = thrust::stable_partition(dp.begin(), dp.end(), _1 < 0.5f) - dp.begin();
  ASSERT_TRUE(hs == ds);
  ASSERT_EQUAL_VEC(bits(to_host(dp)), bits(hp));
}

static void TestSetOperationsSimple() {
  // testing/set_difference.cu:70-80, set_intersection.cu:71-81, set_symmetric_difference.cu:70-80,
  // set_union.cu:71-106, set_union_descending.cu:7-18 and the *_by_key.cu simple tests
  g_test = "SetOperationsSimple";
  {
    thrust::device_vector<int> a(hv<int>({0, 2, 4, 5})), b(hv<int>({0, 3, 3, 4, 6})), r(9);
    r.resize(thrust::set_difference(a.begin(), a.end(), b.begin(), b.end(), r.begin()) - r.begin());
    ASSERT_EQUAL_VEC(to_host(r), hv<int>({2, 5}));
  }
  {
    thrust::device_vector<int> a(hv<int>({0, 2, 4})), b(hv<int>({0, 3, 3, 4})), r(7);
    r.resize(thrust::set_intersection(thrust::device, a.begin(), a.end(), b.begin(), b.end(), r.begin()) - r.begin());
    ASSERT_EQUAL_VEC(to_host(r), hv<int>({0, 4}));
    r.resize(7);
    r.resize(thrust::set_union(a.begin(), a.end(), b.begin(), b.end(), r.begin()) - r.begin());
    ASSERT_EQUAL_VEC(to_host(r), hv<int>({0, 2, 3, 3, 4}));
    thrust::host_vector<int> ha = to_host(a), hb = to_host(b), hr(7);
    hr.resize(thrust::set_union(ha.begin(), ha.end(), hb.begin(), hb.end(), hr.begin()) - hr.begin());
    ASSERT_EQUAL_VEC(hr, hv<int>({0, 2, 3, 3, 4}));
  }
  {
    thrust::device_vector<int> a(hv<int>({0, 2, 2})), b(hv<int>({0, 2, 2, 2, 3})), r(8);
    r.resize(thrust::set_union(a.begin(), a.end(), b.begin(), b.end(), r.begin()) - r.begin());
    ASSERT_EQUAL_VEC(to_host(r), hv<int>({0, 2, 2, 2, 3}));
  }
  {
    thrust::device_vector<int> a(hv<int>({0, 2, 4, 6})), b(hv<int>({0, 3, 3, 4, 7})), r(9);
    r.resize(thrust::set_symmetric_difference(a.begin(), a.end(), b.begin(), b.end(), r.begin()) - r.begin());
    ASSERT_EQUAL_VEC(to_host(r), hv<int>({2, 3, 3, 6, 7}));
  }
  {
    thrust::device_vector<int> a(hv<int>({4, 2, 0})), b(hv<int>({4, 3, 3, 0})), r(7);
    r.resize(thrust::set_union(a.begin(), a.end(), b.begin(), b.end(), r.begin(), thrust::greater<int>()) - r.begin());
    ASSERT_EQUAL_VEC(to_host(r), hv<int>({4, 3, 3, 2, 0}));
  }
  {
    thrust::device_vector<int> ak(hv<int>({0, 2, 4})), av(hv<int>({0, 0, 0}));
    thrust::device_vector<int> bk(hv<int>({0, 3, 3, 4})), bv(hv<int>({1, 1, 1, 1})), rk(7), rv(7);
    auto e = thrust::set_union_by_key(ak.begin(), ak.end(), bk.begin(), bk.end(), av.begin(), bv.begin(), rk.begin(), rv.begin());
    ASSERT_TRUE(e.first - rk.begin() == 5 && e.second - rv.begin() == 5);
    rk.resize(5); rv.resize(5);
    ASSERT_EQUAL_VEC(to_host(rk), hv<int>({0, 2, 3, 3, 4}));
    ASSERT_EQUAL_VEC(to_host(rv), hv<int>({0, 0, 1, 1, 0}));
    rk.resize(7); rv.resize(7);
    e = thrust::set_intersection_by_key(ak.begin(), ak.end(), bk.begin(), bk.end(), av.begin(), rk.begin(), rv.begin());
    ASSERT_TRUE(e.first - rk.begin() == 2);
    rk.resize(2); rv.resize(2);
    ASSERT_EQUAL_VEC(to_host(rk), hv<int>({0, 4}));
    ASSERT_EQUAL_VEC(to_host(rv), hv<int>({0, 0}));
  }
  {
    thrust::device_vector<int> ak(hv<int>({6, 4, 2, 0})), av(hv<int>({0, 0, 0, 0}));
    thrust::device_vector<int> bk(hv<int>({7, 4, 3, 3, 0})), bv(hv<int>({1, 1, 1, 1, 1})), rk(9), rv(9);
    auto e = thrust::set_symmetric_difference_by_key(thrust::device, ak.begin(), ak.end(), bk.begin(), bk.end(), av.begin(),
                                                     bv.begin(), rk.begin(), rv.begin(), thrust::greater<int>());
    ASSERT_TRUE(e.first - rk.begin() == 5);
    rk.resize(5); rv.resize(5);
    ASSERT_EQUAL_VEC(to_host(rk), hv<int>({7, 6, 3, 3, 2}));
    ASSERT_EQUAL_VEC(to_host(rv), hv<int>({1, 0, 1, 1, 0}));
    rk.resize(9); rv.resize(9);
    e = thrust::set_difference_by_key(ak.begin(), ak.end(), bk.begin(), bk.end(), av.begin(), bv.begin(), rk.begin(),
                                      rv.begin(), thrust::greater<int>());
    ASSERT_TRUE(e.first - rk.begin() == 2);
    rk.resize(2);
    ASSERT_EQUAL_VEC(to_host(rk), hv<int>({6, 2}));
  }
}

static void TestSortSimple() {  // testing/sort.cu:43-76
  g_test = "SortSimple";
  thrust::device_vector<int> d(hv<int>({1, 3, 6, 5, 2, 0, 4}));
  thrust::sort(d.begin(), d.end());
  ASSERT_EQUAL_VEC(to_host(d), hv<int>({0, 1, 2, 3, 4, 5, 6}));
  thrust::sort(d.begin(), d.end(), thrust::greater<int>());
  ASSERT_EQUAL_VEC(to_host(d), hv<int>({6, 5, 4, 3, 2, 1, 0}));
  thrust::stable_sort(thrust::device, d.begin(), d.end(), thrust::less<int>());
  ASSERT_EQUAL_VEC(to_host(d), hv<int>({0, 1, 2, 3, 4, 5, 6}));
}

static void TestSortByKeySimple() {  // testing/sort_by_key.cu:47-85, stable_sort_by_key.cu:51-95
  g_test = "SortByKeySimple";
  thrust::device_vector<int> keys(hv<int>({1, 3, 6, 5, 2, 0, 4}));
  thrust::device_vector<int> vals(hv<int>({0, 1, 2, 3, 4, 5, 6}));
  thrust::sort_by_key(keys.begin(), keys.end(), vals.begin());
  ASSERT_EQUAL_VEC(to_host(keys), hv<int>({0, 1, 2, 3, 4, 5, 6}));
  ASSERT_EQUAL_VEC(to_host(vals), hv<int>({5, 0, 4, 1, 6, 3, 2}));
  // stability: equal keys keep the order of their values
  thrust::device_vector<int> k2(hv<int>({2, 1, 2, 1, 2, 1, 0, 0, 1}));
  thrust::device_vector<int> v2(hv<int>({0, 1, 2, 3, 4, 5, 6, 7, 8}));
  thrust::stable_sort_by_key(k2.begin(), k2.end(), v2.begin());
  ASSERT_EQUAL_VEC(to_host(k2), hv<int>({0, 0, 1, 1, 1, 1, 2, 2, 2}));
  ASSERT_EQUAL_VEC(to_host(v2), hv<int>({6, 7, 1, 3, 5, 8, 0, 2, 4}));
  thrust::stable_sort_by_key(k2.begin(), k2.end(), v2.begin(), thrust::greater<int>());
  ASSERT_EQUAL_VEC(to_host(k2), hv<int>({2, 2, 2, 1, 1, 1, 1, 0, 0}));
  ASSERT_EQUAL_VEC(to_host(v2), hv<int>({0, 2, 4, 1, 3, 5, 8, 6, 7}));
}

static void TestReduceByKeySimple() {  // testing/reduce_by_key.cu:16-112
  g_test = "ReduceByKeySimple";
  thrust::device_vector<int> keys(hv<int>({11, 11, 21, 20, 21, 21, 21, 37, 37}));
  thrust::device_vector<int> vals(hv<int>({0, 1, 2, 3, 4, 5, 6, 7, 8}));
  thrust::device_vector<int> ok(9), ov(9);
  auto ends = thrust::reduce_by_key(keys.begin(), keys.end(), vals.begin(), ok.begin(), ov.begin());
  ASSERT_TRUE(ends.first - ok.begin() == 5 && ends.second - ov.begin() == 5);
  ok.resize(5); ov.resize(5);
  ASSERT_EQUAL_VEC(to_host(ok), hv<int>({11, 21, 20, 21, 37}));
  ASSERT_EQUAL_VEC(to_host(ov), hv<int>({1, 2, 3, 15, 15}));
  ok.resize(9); ov.resize(9);
  ends = thrust::reduce_by_key(keys.begin(), keys.end(), vals.begin(), ok.begin(), ov.begin(),
                               thrust::equal_to<int>(), thrust::plus<int>());
  ASSERT_TRUE(ends.first - ok.begin() == 5);
  ok.resize(5); ov.resize(5);
  ASSERT_EQUAL_VEC(to_host(ov), hv<int>({1, 2, 3, 15, 15}));
}

static void TestUniqueSimple() {  // testing/unique.cu:105-142
  g_test = "UniqueSimple";
  thrust::device_vector<int> d(hv<int>({11, 11, 12, 20, 29, 21, 21, 31, 31, 37}));
  auto e = thrust::unique(d.begin(), d.end());
  ASSERT_TRUE(e - d.begin() == 7);
  d.resize(7);
  ASSERT_EQUAL_VEC(to_host(d), hv<int>({11, 12, 20, 29, 21, 31, 37}));
  thrust::device_vector<int> src(hv<int>({11, 11, 12, 20, 29, 21, 21, 31, 31, 37})), out(10);
  auto e2 = thrust::unique_copy(src.begin(), src.end(), out.begin());
  ASSERT_TRUE(e2 - out.begin() == 7);
}

static void TestUniqueByKeySimple() {  // testing/unique_by_key.cu:160-253
  g_test = "UniqueByKeySimple";
  thrust::device_vector<int> keys(hv<int>({11, 11, 21, 20, 21, 21, 21, 37, 37}));
  thrust::device_vector<int> vals(hv<int>({0, 1, 2, 3, 4, 5, 6, 7, 8}));
  thrust::device_vector<int> ok(9), ov(9);
  auto ends = thrust::unique_by_key_copy(keys.begin(), keys.end(), vals.begin(), ok.begin(), ov.begin());
  ASSERT_TRUE(ends.first - ok.begin() == 5 && ends.second - ov.begin() == 5);
  ok.resize(5); ov.resize(5);
  ASSERT_EQUAL_VEC(to_host(ok), hv<int>({11, 21, 20, 21, 37}));
  ASSERT_EQUAL_VEC(to_host(ov), hv<int>({0, 2, 3, 4, 7}));
  auto ends2 = thrust::unique_by_key(keys.begin(), keys.end(), vals.begin());
  ASSERT_TRUE(ends2.first - keys.begin() == 5);
  keys.resize(5); vals.resize(5);
  ASSERT_EQUAL_VEC(to_host(keys), hv<int>({11, 21, 20, 21, 37}));
  ASSERT_EQUAL_VEC(to_host(vals), hv<int>({0, 2, 3, 4, 7}));
}

static void TestCopyIfSimple() {  // testing/copy.cu:252-269, :378-397
  g_test = "CopyIfSimple";
  thrust::device_vector<int> v(hv<int>({0, 1, 2, 3, 4})), dest(5, 10);
  auto e = thrust::copy_if(v.begin(), v.end(), dest.begin(), thrust::identity<int>());  // "is_true"
  ASSERT_TRUE(e - dest.begin() == 4);
  dest.resize(4);
  ASSERT_EQUAL_VEC(to_host(dest), hv<int>({1, 2, 3, 4}));
  // stencil form
  thrust::device_vector<int> st(hv<int>({1, 0, 1, 0, 1})), dest2(5, 0);
  auto e2 = thrust::copy_if(v.begin(), v.end(), st.begin(), dest2.begin(), thrust::identity<int>());
  ASSERT_TRUE(e2 - dest2.begin() == 3);
  dest2.resize(3);
  ASSERT_EQUAL_VEC(to_host(dest2), hv<int>({0, 2, 4}));
}

static void TestStablePartitionSimple() {  // testing/partition.cu:158-182 with is_even as a stencil
  g_test = "StablePartitionSimple";
  thrust::device_vector<int> data(hv<int>({1, 2, 1, 3, 2}));
  // is_even(x) expressed through a stencil of parities and "== 0"
  thrust::device_vector<int> parity(hv<int>({1, 0, 1, 1, 0}));
  auto mid = thrust::stable_partition(data.begin(), data.end(), parity.begin(), _1 == 0);
  ASSERT_TRUE(mid - data.begin() == 2);
  ASSERT_EQUAL_VEC(to_host(data), hv<int>({2, 2, 1, 1, 3}));
  // predicate on the data itself
  thrust::device_vector<int> d2(hv<int>({5, 1, 7, 2, 9, 3}));
  auto m2 = thrust::partition(d2.begin(), d2.end(), _1 < 4);
  ASSERT_TRUE(m2 - d2.begin() == 3);
  ASSERT_EQUAL_VEC(to_host(d2), hv<int>({1, 2, 3, 5, 7, 9}));
  thrust::device_vector<int> src(hv<int>({5, 1, 7, 2, 9, 3})), t(6), f(6);
  auto ends = thrust::stable_partition_copy(src.begin(), src.end(), t.begin(), f.begin(), _1 >= 5);
  ASSERT_TRUE(ends.first - t.begin() == 3 && ends.second - f.begin() == 3);
  t.resize(3); f.resize(3);
  ASSERT_EQUAL_VEC(to_host(t), hv<int>({5, 7, 9}));
  ASSERT_EQUAL_VEC(to_host(f), hv<int>({1, 2, 3}));
}

static void TestMergeSimple() {  // testing/merge.cu:11-38
  g_test = "MergeSimple";
  thrust::device_vector<int> a(hv<int>({0, 2, 4})), b(hv<int>({0, 3, 3, 4})), r(7);
  auto e = thrust::merge(a.begin(), a.end(), b.begin(), b.end(), r.begin());
  ASSERT_TRUE(e - r.begin() == 7);
  ASSERT_EQUAL_VEC(to_host(r), hv<int>({0, 0, 2, 3, 3, 4, 4}));
}

static void TestMergeByKeySimple() {  // testing/merge_by_key.cu:10-45
  g_test = "MergeByKeySimple";
  thrust::device_vector<int> ak(hv<int>({0, 2, 4})), av(hv<int>({13, 7, 42}));
  thrust::device_vector<int> bk(hv<int>({0, 3, 3, 4})), bv(hv<int>({42, 42, 7, 13}));
  thrust::device_vector<int> rk(7), rv(7);
  auto ends = thrust::merge_by_key(ak.begin(), ak.end(), bk.begin(), bk.end(), av.begin(), bv.begin(),
                                   rk.begin(), rv.begin());
  ASSERT_TRUE(ends.first - rk.begin() == 7 && ends.second - rv.begin() == 7);
  ASSERT_EQUAL_VEC(to_host(rk), hv<int>({0, 0, 2, 3, 3, 4, 4}));
  ASSERT_EQUAL_VEC(to_host(rv), hv<int>({13, 42, 7, 42, 7, 42, 13}));  // ties: first range first
}

// ================================================================ part 2: host vs device
template <typename T>
static void DifferentialForType(const char* name) {
  std::string label = std::string("Differential<") + name + ">";
  g_test = label.c_str();
  for (size_t n : kSizes) {
    thrust::host_vector<T> h = random_integers<T>(n, 7, 0);
    thrust::device_vector<T> d = h;
    // reduce (wraps in T on both systems for integers)
    const T init = (T)13;
    if (std::is_integral<T>::value) {
      using U = typename std::conditional<std::is_integral<T>::value, typename std::make_unsigned<
                typename std::conditional<std::is_integral<T>::value, T, int>::type>::type, T>::type;
      U acc = (U)init;
      for (size_t i = 0; i < n; ++i) acc = (U)(acc + (U)h[i]);
      ASSERT_TRUE(thrust::reduce(d.begin(), d.end(), init) == (T)acc);
    }
    // sort / stable_sort
    thrust::host_vector<T> hs = h;
    thrust::device_vector<T> ds = d;
    thrust::sort(hs.begin(), hs.end());
    thrust::sort(ds.begin(), ds.end());
    ASSERT_EQUAL_VEC(to_host(ds), hs);
    hs = h; ds = d;
    thrust::sort(hs.begin(), hs.end(), thrust::greater<T>());
    thrust::sort(ds.begin(), ds.end(), thrust::greater<T>());
    ASSERT_EQUAL_VEC(to_host(ds), hs);
    // sort_by_key with duplicate-heavy keys: values reveal stability
    thrust::host_vector<T> hk = random_integers<T>(n, 9, 17);
    thrust::host_vector<unsigned int> hval(n);
    for (size_t i = 0; i < n; ++i) hval[i] = (unsigned int)i;
    thrust::device_vector<T> dk = hk;
    thrust::device_vector<unsigned int> dval = hval;
    thrust::stable_sort_by_key(hk.begin(), hk.end(), hval.begin());
    thrust::stable_sort_by_key(dk.begin(), dk.end(), dval.begin());
    ASSERT_EQUAL_VEC(to_host(dk), hk);
    ASSERT_EQUAL_VEC(to_host(dval), hval);
    // unique / unique_by_key on the sorted keys
    thrust::host_vector<T> hu = hk;
    thrust::device_vector<T> du = dk;
    hu.resize(thrust::unique(hu.begin(), hu.end()) - hu.begin());
    du.resize(thrust::unique(du.begin(), du.end()) - du.begin());
    ASSERT_EQUAL_VEC(to_host(du), hu);
    // reduce_by_key
    thrust::host_vector<T> hko(n);
    thrust::host_vector<unsigned int> hvo(n);
    thrust::device_vector<T> dko(n);
    thrust::device_vector<unsigned int> dvo(n);
    auto he = thrust::reduce_by_key(hk.begin(), hk.end(), hval.begin(), hko.begin(), hvo.begin());
    auto de = thrust::reduce_by_key(dk.begin(), dk.end(), dval.begin(), dko.begin(), dvo.begin());
    ASSERT_TRUE((he.first - hko.begin()) == (de.first - dko.begin()));
    hko.resize(he.first - hko.begin()); hvo.resize(hko.size());
    dko.resize(hko.size()); dvo.resize(hko.size());
    ASSERT_EQUAL_VEC(to_host(dko), hko);
    ASSERT_EQUAL_VEC(to_host(dvo), hvo);
    // scans (integers: exact)
    if (std::is_integral<T>::value) {
      thrust::host_vector<T> ho(n);
      thrust::device_vector<T> dout(n);
      thrust::inclusive_scan(h.begin(), h.end(), ho.begin());
      thrust::inclusive_scan(d.begin(), d.end(), dout.begin());
      ASSERT_EQUAL_VEC(to_host(dout), ho);
      thrust::exclusive_scan(h.begin(), h.end(), ho.begin(), (T)11);
      thrust::exclusive_scan(d.begin(), d.end(), dout.begin(), (T)11);
      ASSERT_EQUAL_VEC(to_host(dout), ho);
    }
    // scan_by_key, count_if, inner_product (integers: exact)
    if (std::is_integral<T>::value) {
      thrust::host_vector<T> hsv = random_integers<T>(n, 41, 0), hso(n);
      thrust::device_vector<T> dsv = hsv, dso(n);
      thrust::inclusive_scan_by_key(hk.begin(), hk.end(), hsv.begin(), hso.begin());
      thrust::inclusive_scan_by_key(dk.begin(), dk.end(), dsv.begin(), dso.begin());
      ASSERT_EQUAL_VEC(to_host(dso), hso);
      thrust::exclusive_scan_by_key(hk.begin(), hk.end(), hsv.begin(), hso.begin(), (T)5);
      thrust::exclusive_scan_by_key(dk.begin(), dk.end(), dsv.begin(), dso.begin(), (T)5);
      ASSERT_EQUAL_VEC(to_host(dso), hso);
      ASSERT_TRUE(thrust::count_if(hk.begin(), hk.end(), _1 < (T)9) == thrust::count_if(dk.begin(), dk.end(), _1 < (T)9));
      ASSERT_TRUE(thrust::count(hk.begin(), hk.end(), (T)3) == thrust::count(dk.begin(), dk.end(), (T)3));
      {  // expected value in unsigned arithmetic (wraps without undefined behaviour)
        using U = typename std::make_unsigned<typename std::conditional<std::is_integral<T>::value, T, int>::type>::type;
        U dot = (U)3;
        for (size_t i = 0; i < n; ++i) dot = (U)(dot + (U)((U)h[i] * (U)hsv[i]));
        ASSERT_TRUE(thrust::inner_product(d.begin(), d.end(), dsv.begin(), (T)3) == (T)dot);
        // transform_reduce / transform scans: negate with plus (testing/transform_scan.cu:253-279)
        U neg = (U)13;
        for (size_t i = 0; i < n; ++i) neg = (U)(neg - (U)h[i]);
        ASSERT_TRUE(thrust::transform_reduce(d.begin(), d.end(), thrust::negate<T>(), (T)13, thrust::plus<T>()) == (T)neg);
        thrust::host_vector<T> hts(n);
        thrust::device_vector<T> dts(n);
        U run = 0;
        for (size_t i = 0; i < n; ++i) { run = (U)(run - (U)h[i]); hts[i] = (T)run; }
        thrust::transform_inclusive_scan(d.begin(), d.end(), dts.begin(), thrust::negate<T>(), thrust::plus<T>());
        ASSERT_EQUAL_VEC(to_host(dts), hts);
        run = (U)11;
        for (size_t i = 0; i < n; ++i) { hts[i] = (T)run; run = (U)(run + (U)((U)h[i] * (U)h[i])); }
        thrust::transform_exclusive_scan(d.begin(), d.end(), dts.begin(), thrust::square<T>(), (T)11, thrust::plus<T>());
        ASSERT_EQUAL_VEC(to_host(dts), hts);
      }
    }
    // remove_if / remove_copy_if / remove against the host system
    {
      thrust::host_vector<T> hr = random_integers<T>(n, 23, 100), hro(n);
      thrust::device_vector<T> dr = hr, dro(n);
      hro.resize(thrust::remove_copy_if(hr.begin(), hr.end(), hro.begin(), _1 >= (T)50) - hro.begin());
      dro.resize(thrust::remove_copy_if(dr.begin(), dr.end(), dro.begin(), _1 >= (T)50) - dro.begin());
      ASSERT_EQUAL_VEC(to_host(dro), hro);
      hr.resize(thrust::remove_if(hr.begin(), hr.end(), _1 < (T)30) - hr.begin());
      dr.resize(thrust::remove_if(dr.begin(), dr.end(), _1 < (T)30) - dr.begin());
      ASSERT_EQUAL_VEC(to_host(dr), hr);
      hr.resize(thrust::remove(hr.begin(), hr.end(), (T)77) - hr.begin());
      dr.resize(thrust::remove(dr.begin(), dr.end(), (T)77) - dr.begin());
      ASSERT_EQUAL_VEC(to_host(dr), hr);
    }
    // copy_if / stable_partition with a threshold predicate
    thrust::host_vector<T> hsel = random_integers<T>(n, 21, 100);
    thrust::device_vector<T> dsel = hsel;
    thrust::host_vector<T> hc(n);
    thrust::device_vector<T> dc(n);
    const T thr = (T)37;
    hc.resize(thrust::copy_if(hsel.begin(), hsel.end(), hc.begin(), _1 < thr) - hc.begin());
    dc.resize(thrust::copy_if(dsel.begin(), dsel.end(), dc.begin(), _1 < thr) - dc.begin());
    ASSERT_EQUAL_VEC(to_host(dc), hc);
    auto hm = thrust::stable_partition(hsel.begin(), hsel.end(), _1 < thr);
    auto dm = thrust::stable_partition(dsel.begin(), dsel.end(), _1 < thr);
    ASSERT_TRUE((hm - hsel.begin()) == (dm - dsel.begin()));
    ASSERT_EQUAL_VEC(to_host(dsel), hsel);
    // merge of two sorted ranges
    thrust::host_vector<T> ha = random_integers<T>(n, 31, 50), hb = random_integers<T>(n / 2 + 1, 33, 50);
    thrust::sort(ha.begin(), ha.end());
    thrust::sort(hb.begin(), hb.end());
    thrust::device_vector<T> da = ha, db = hb;
    thrust::host_vector<T> hr(ha.size() + hb.size());
    thrust::device_vector<T> dr(ha.size() + hb.size());
    thrust::merge(ha.begin(), ha.end(), hb.begin(), hb.end(), hr.begin());
    thrust::merge(da.begin(), da.end(), db.begin(), db.end(), dr.begin());
    ASSERT_EQUAL_VEC(to_host(dr), hr);
    // the four set operations on the same sorted ranges (values drawn from 50 keys: long runs)
    {
      thrust::host_vector<T> hs(ha.size() + hb.size());
      thrust::device_vector<T> ds(ha.size() + hb.size());
      size_t hn = thrust::set_difference(ha.begin(), ha.end(), hb.begin(), hb.end(), hs.begin()) - hs.begin();
      size_t dn = thrust::set_difference(da.begin(), da.end(), db.begin(), db.end(), ds.begin()) - ds.begin();
      ASSERT_TRUE(hn == dn);
      ASSERT_TRUE(std::equal(hs.begin(), hs.begin() + hn, to_host(ds).begin()));
      hn = thrust::set_intersection(ha.begin(), ha.end(), hb.begin(), hb.end(), hs.begin()) - hs.begin();
      dn = thrust::set_intersection(da.begin(), da.end(), db.begin(), db.end(), ds.begin()) - ds.begin();
      ASSERT_TRUE(hn == dn);
      ASSERT_TRUE(std::equal(hs.begin(), hs.begin() + hn, to_host(ds).begin()));
      hn = thrust::set_symmetric_difference(ha.begin(), ha.end(), hb.begin(), hb.end(), hs.begin()) - hs.begin();
      dn = thrust::set_symmetric_difference(da.begin(), da.end(), db.begin(), db.end(), ds.begin()) - ds.begin();
      ASSERT_TRUE(hn == dn);
      ASSERT_TRUE(std::equal(hs.begin(), hs.begin() + hn, to_host(ds).begin()));
      hn = thrust::set_union(ha.begin(), ha.end(), hb.begin(), hb.end(), hs.begin()) - hs.begin();
      dn = thrust::set_union(da.begin(), da.end(), db.begin(), db.end(), ds.begin()) - ds.begin();
      ASSERT_TRUE(hn == dn);
      ASSERT_TRUE(std::equal(hs.begin(), hs.begin() + hn, to_host(ds).begin()));
      // by key: the values name the side and the index of every kept element
      thrust::host_vector<int> hva(ha.size()), hvb(hb.size()), hvo(ha.size() + hb.size());
      for (size_t i = 0; i < hva.size(); ++i) hva[i] = (int)i;
      for (size_t i = 0; i < hvb.size(); ++i) hvb[i] = -(int)i - 1;
      thrust::device_vector<int> dva = hva, dvb = hvb, dvo(ha.size() + hb.size());
      auto he = thrust::set_union_by_key(ha.begin(), ha.end(), hb.begin(), hb.end(), hva.begin(), hvb.begin(), hs.begin(), hvo.begin());
      auto de = thrust::set_union_by_key(da.begin(), da.end(), db.begin(), db.end(), dva.begin(), dvb.begin(), ds.begin(), dvo.begin());
      ASSERT_TRUE((he.first - hs.begin()) == (de.first - ds.begin()));
      ASSERT_TRUE(std::equal(hvo.begin(), hvo.begin() + (he.second - hvo.begin()), to_host(dvo).begin()));
      he = thrust::set_symmetric_difference_by_key(ha.begin(), ha.end(), hb.begin(), hb.end(), hva.begin(), hvb.begin(), hs.begin(), hvo.begin());
      de = thrust::set_symmetric_difference_by_key(da.begin(), da.end(), db.begin(), db.end(), dva.begin(), dvb.begin(), ds.begin(), dvo.begin());
      ASSERT_TRUE((he.first - hs.begin()) == (de.first - ds.begin()));
      ASSERT_TRUE(std::equal(hvo.begin(), hvo.begin() + (he.second - hvo.begin()), to_host(dvo).begin()));
      he = thrust::set_intersection_by_key(ha.begin(), ha.end(), hb.begin(), hb.end(), hva.begin(), hs.begin(), hvo.begin());
      de = thrust::set_intersection_by_key(da.begin(), da.end(), db.begin(), db.end(), dva.begin(), ds.begin(), dvo.begin());
      ASSERT_TRUE((he.first - hs.begin()) == (de.first - ds.begin()));
      ASSERT_TRUE(std::equal(hvo.begin(), hvo.begin() + (he.second - hvo.begin()), to_host(dvo).begin()));
      he = thrust::set_difference_by_key(ha.begin(), ha.end(), hb.begin(), hb.end(), hva.begin(), hvb.begin(), hs.begin(), hvo.begin());
      de = thrust::set_difference_by_key(da.begin(), da.end(), db.begin(), db.end(), dva.begin(), dvb.begin(), ds.begin(), dvo.begin());
      ASSERT_TRUE((he.first - hs.begin()) == (de.first - ds.begin()));
      ASSERT_TRUE(std::equal(hvo.begin(), hvo.begin() + (he.second - hvo.begin()), to_host(dvo).begin()));
    }
  }
}

static void TestFloatSortTotalOrder() {
  g_test = "FloatSortTotalOrder";
  // -0.0 sorts before +0.0 (radix order on the encoded bits), as the reference's
  // sequential radix sort does (stable_radix_sort.inl:115-125)
  thrust::device_vector<float> d(hv<float>({0.0f, -0.0f, 1.0f, -1.0f, 0.0f, -0.0f}));
  thrust::sort(d.begin(), d.end());
  thrust::host_vector<float> h = d;
  const uint32_t expect[6] = {0xBF800000u, 0x80000000u, 0x80000000u, 0u, 0u, 0x3F800000u};
  for (int i = 0; i < 6; ++i) {
    uint32_t bits;
    std::memcpy(&bits, &h[i], 4);
    ASSERT_TRUE(bits == expect[i]);
  }
}

// ================================================================ part 3: policies, dispatch, memory
// A user policy derived from device_execution_policy intercepts an algorithm by overload,
// as in the reference's examples/minimal_custom_backend.cu:17-37 and
// testing/unittest/special_types.h:131-166 (my_system / validate_dispatch).
struct my_system : thrust::device_execution_policy<my_system> {
  mutable bool dispatched = false;
};
template <typename It>
void sort(my_system& sys, It first, It last) {
  sys.dispatched = true;
}
template <typename It, typename T>
T reduce(my_system& sys, It, It, T init) {
  sys.dispatched = true;
  return init;
}

static void TestDispatch() {
  g_test = "Dispatch";
  thrust::device_vector<int> d(hv<int>({3, 1, 2}));
  my_system sys;
  thrust::sort(sys, d.begin(), d.end());
  ASSERT_TRUE(sys.dispatched);
  ASSERT_EQUAL_VEC(to_host(d), hv<int>({3, 1, 2}));  // the user's overload ran, not ours
  my_system sys2;
  ASSERT_TRUE(thrust::reduce(sys2, d.begin(), d.end(), 42) == 42 && sys2.dispatched);
  // a derived policy without overloads falls through to the device system
  my_system sys3;
  thrust::stable_sort(sys3, d.begin(), d.end());
  ASSERT_TRUE(!sys3.dispatched);
  ASSERT_EQUAL_VEC(to_host(d), hv<int>({1, 2, 3}));
}

static void TestPoliciesAndRawPointers() {
  g_test = "Policies";
  thrust::device_vector<int> d(hv<int>({5, 4, 3, 2, 1}));
  int* raw = thrust::raw_pointer_cast(d.data());
  // raw device pointers need an explicit device policy
  thrust::sort(thrust::device, raw, raw + 5);
  ASSERT_EQUAL_VEC(to_host(d), hv<int>({1, 2, 3, 4, 5}));
  ASSERT_TRUE(thrust::reduce(thrust::hip::par, raw, raw + 5) == 15);
  ASSERT_TRUE(thrust::reduce(thrust::hip::par.on(nullptr), d.begin(), d.end(), 1) == 16);
  // host policies and containers run on the host system
  std::vector<int> hvec = {3, 1, 2};
  thrust::sort(thrust::host, hvec.begin(), hvec.end());
  ASSERT_TRUE(hvec[0] == 1 && hvec[2] == 3);
  ASSERT_TRUE(thrust::reduce(thrust::seq, hvec.begin(), hvec.end()) == 6);
  thrust::device_ptr<int> p = thrust::device_pointer_cast(raw);
  ASSERT_TRUE(thrust::reduce(p, p + 5) == 15);
}

static void TestDeviceVector() {
  g_test = "DeviceVector";
  thrust::device_vector<int> a(4, 7);
  ASSERT_TRUE(a.size() == 4 && (int)a[0] == 7 && (int)a[3] == 7);
  a[1] = 42;
  ASSERT_TRUE((int)a[1] == 42);
  a[1] += 1;
  ASSERT_TRUE((int)a[1] == 43);
  thrust::device_vector<int> b = a;  // device to device
  b.resize(6);                       // new elements are value-initialised
  ASSERT_TRUE(b.size() == 6 && (int)b[1] == 43 && (int)b[5] == 0);
  thrust::host_vector<int> h = b;
  ASSERT_TRUE(h.size() == 6 && h[0] == 7 && h[1] == 43);
  thrust::device_vector<int> c(h.begin(), h.end());
  ASSERT_TRUE(c == b);
  c.push_back(9);
  ASSERT_TRUE(c.size() == 7 && (int)c.back() == 9);
  thrust::fill(c.begin(), c.end(), 3);
  ASSERT_TRUE(thrust::reduce(c.begin(), c.end()) == 21);
  thrust::copy(h.begin(), h.end(), c.begin());  // host to device
  ASSERT_TRUE((int)c[1] == 43);
  std::vector<int> out(6);
  thrust::copy(b.begin(), b.end(), out.begin());  // device to host
  ASSERT_TRUE(out[1] == 43 && out[5] == 0);
  thrust::device_vector<double> e;
  ASSERT_TRUE(e.empty() && thrust::reduce(e.begin(), e.end()) == 0.0);
  thrust::device_vector<int> moved(std::move(c));
  ASSERT_TRUE(moved.size() == 7 && c.size() == 0);
  a.swap(b);
  ASSERT_TRUE(a.size() == 6 && b.size() == 4);
}

static void TestOutOfMemoryThrows() {  // testing/out_of_memory_recovery.cu:24-34
  g_test = "OutOfMemory";
  bool threw = false;
  try {
    thrust::device_vector<uint32_t> y(0x00ffffffffffffffull);
  } catch (const std::bad_alloc&) {
    threw = true;
  }
  ASSERT_TRUE(threw);
  // the system stays usable afterwards
  thrust::device_vector<int> ok(hv<int>({2, 1}));
  thrust::sort(ok.begin(), ok.end());
  ASSERT_EQUAL_VEC(to_host(ok), hv<int>({1, 2}));
}

static void TestTempArenaReuse() {
  g_test = "TempArena";
  thrust::device_vector<int> d(1 << 20, 1);
  (void)thrust::reduce(d.begin(), d.end());
  const size_t held = thrust_amd_temp_bytes_held();
  for (int i = 0; i < 10; ++i) (void)thrust::reduce(d.begin(), d.end());
  ASSERT_TRUE(thrust_amd_temp_bytes_held() == held);  // steady state: no new allocations
  ASSERT_TRUE(thrust_amd_temp_trim() == 0);
  ASSERT_TRUE(thrust_amd_temp_bytes_held() == 0);
}

// A block cache in the role of the reference's examples/cuda/custom_temporary_allocation.cu:
// freed blocks are kept by size and handed out again.  `skew` shifts every pointer it returns,
// to show that the library does not rely on the allocator's alignment.
struct CachingTempAllocator {
  typedef char value_type;
  std::multimap<std::ptrdiff_t, char*> free_blocks;
  std::map<char*, std::ptrdiff_t> live;
  int fresh = 0, reused = 0, returned = 0;
  std::ptrdiff_t skew = 0;
  char* allocate(std::ptrdiff_t n) {
    char* block = nullptr;
    auto hit = free_blocks.find(n);
    if (hit != free_blocks.end()) {
      block = hit->second;
      free_blocks.erase(hit);
      ++reused;
    } else {
      block = thrust::device_malloc<char>((std::size_t)(n + skew)).get();
      ++fresh;
    }
    live[block + skew] = n;
    return block + skew;
  }
  void deallocate(char* p, std::size_t n) {
    auto it = live.find(p);
    if (it == live.end() || it->second != (std::ptrdiff_t)n) throw std::runtime_error("not a live block of this allocator");
    live.erase(it);
    free_blocks.insert(std::make_pair((std::ptrdiff_t)n, p - skew));
    ++returned;
  }
  ~CachingTempAllocator() {
    for (auto& b : free_blocks) thrust::device_free(thrust::device_pointer_cast(b.second));
  }
};

// The same interface handing out device_ptr<char>, as an allocator built on thrust::device_malloc would.
struct FancyPointerAllocator {
  typedef char value_type;
  int calls = 0;
  thrust::device_ptr<char> allocate(std::size_t n) { ++calls; return thrust::device_malloc<char>(n); }
  void deallocate(thrust::device_ptr<char> p, std::size_t) { --calls; thrust::device_free(p); }
};

struct FailingAllocator {
  typedef char value_type;
  char* allocate(std::size_t) { throw std::bad_alloc(); }
  void deallocate(char*, std::size_t) {}
};

static void TestCustomTemporaryAllocation() {  // examples/cuda/custom_temporary_allocation.cu:142-186
  g_test = "CustomTemporaryAllocation";
  const size_t n = 1 << 16;
  thrust::host_vector<int> h = random_integers<int>(n, 3, 0);
  thrust::host_vector<int> sorted = h;
  thrust::sort(sorted.begin(), sorted.end());
  for (std::ptrdiff_t skew : {0, 8}) {
    CachingTempAllocator alloc;
    alloc.skew = skew;
    ASSERT_TRUE(thrust_amd_temp_trim() == 0);
    for (int round = 0; round < 3; ++round) {
      thrust::device_vector<int> d = h;
      thrust::sort(thrust::hip::par(alloc), d.begin(), d.end());
      ASSERT_EQUAL_VEC(to_host(d), sorted);
    }
    ASSERT_TRUE(alloc.fresh == 1 && alloc.reused == 2 && alloc.returned == 3 && alloc.live.empty());
    ASSERT_TRUE(thrust_amd_temp_bytes_held() == 0);  // the library's own arena was not touched
    // other algorithms through the same policy, also bound to a stream
    thrust::device_vector<int> d = h, out(n);
    long long total = 0;
    for (size_t i = 0; i < n; ++i) total += h[i];
    ASSERT_TRUE(thrust::reduce(thrust::hip::par(alloc).on(nullptr), d.begin(), d.end(), 0) == (int)total);
    thrust::inclusive_scan(thrust::hip::par(alloc), d.begin(), d.end(), out.begin());
    thrust::host_vector<int> hs(n);
    thrust::inclusive_scan(h.begin(), h.end(), hs.begin());
    ASSERT_EQUAL_VEC(to_host(out), hs);
    thrust::host_vector<int> hc(n);
    hc.resize(thrust::copy_if(h.begin(), h.end(), hc.begin(), _1 < 1000) - hc.begin());
    out.resize(thrust::copy_if(thrust::hip::par(alloc), d.begin(), d.end(), out.begin(), _1 < 1000) - out.begin());
    ASSERT_EQUAL_VEC(to_host(out), hc);
    thrust::device_vector<int> keys = h, vals(n, 1), ko(n), vo(n);
    thrust::sort_by_key(thrust::hip::par(alloc), keys.begin(), keys.end(), vals.begin());
    auto ends = thrust::reduce_by_key(thrust::hip::par(alloc), keys.begin(), keys.end(), vals.begin(), ko.begin(), vo.begin());
    ASSERT_TRUE(thrust::reduce(thrust::hip::par(alloc), vo.begin(), ends.second, 0) == (int)n);
    ASSERT_TRUE(alloc.live.empty() && alloc.returned == alloc.fresh + alloc.reused);
    ASSERT_TRUE(thrust_amd_temp_bytes_held() == 0);
  }
  FancyPointerAllocator fancy;
  thrust::device_vector<int> d = h;
  thrust::sort(thrust::hip::par(fancy), d.begin(), d.end());
  ASSERT_EQUAL_VEC(to_host(d), sorted);
  ASSERT_TRUE(fancy.calls == 0);
  // an allocator that throws: the exception reaches the caller and the data is untouched
  FailingAllocator failing;
  d = h;
  bool threw = false;
  try {
    thrust::sort(thrust::hip::par(failing), d.begin(), d.end());
  } catch (const std::bad_alloc&) {
    threw = true;
  }
  ASSERT_TRUE(threw);
  ASSERT_EQUAL_VEC(to_host(d), h);
}

// thrust::async: results equal the synchronous algorithms; the stream of the result follows
// .on(stream) / .after(...) as testing/async_reduce.cu:773-990 checks; independent work
// overlaps on streams of its own (testing/async_sort.cu, async_copy.cu, async/inclusive_scan).
static void TestAsyncAlgorithms() {
  g_test = "AsyncAlgorithms";
  const size_t n = (1 << 20) + 17;
  thrust::host_vector<int> h = random_integers<int>(n, 5, 0);
  thrust::device_vector<int> d0 = h, d1 = h, d2 = h, d3 = h;
  long long total = 0;
  for (size_t i = 0; i < n; ++i) total += h[i];
  const int expect = (int)total;

  // four independent reductions in flight, each on a stream of its own
  auto f0a = thrust::async::reduce(d0.begin(), d0.end());
  auto f0b = thrust::async::reduce(thrust::device, d1.begin(), d1.end());
  auto f0c = thrust::async::reduce(thrust::device, d2.begin(), d2.end(), 0);
  auto f0d = thrust::async::reduce(thrust::device, d3.begin(), d3.end(), 7, thrust::plus<int>());
  ASSERT_TRUE(f0a.valid_stream() && f0b.valid_stream() && f0a.valid_content());
  ASSERT_TRUE(f0a.stream().native_handle() != f0b.stream().native_handle());
  ASSERT_TRUE(f0a.get() == expect && f0b.get() == expect && f0c.get() == expect && f0d.get() == expect + 7);
  ASSERT_TRUE(f0a.ready());
  ASSERT_TRUE(f0a.extract() == expect);  // the value stays available

  // .after: runs on the first dependency's stream once every dependency has finished
  auto g0 = thrust::async::reduce(d0.begin(), d0.end());
  void* g0_stream = g0.stream().native_handle();
  auto g1 = thrust::async::reduce(thrust::device.after(g0), d0.begin(), d0.end());
  ASSERT_TRUE(g1.stream().native_handle() == g0_stream);
  auto g2 = thrust::async::reduce(thrust::device.after(g1, f0b), d0.begin(), d0.end());
  ASSERT_TRUE(g2.stream().native_handle() == g0_stream);
  ASSERT_TRUE(g2.get() == expect && g0.get() == expect);

  // .on(stream) wins over the dependencies' streams
  void* user_stream = nullptr;
  ASSERT_TRUE(thrust_amd_stream_create(&user_stream) == 0);
  auto k0 = thrust::async::reduce(thrust::device.on(user_stream), d0.begin(), d0.end());
  ASSERT_TRUE(k0.stream().native_handle() == user_stream);
  auto k1 = thrust::async::reduce(thrust::device.on(user_stream).after(g2), d0.begin(), d0.end());
  ASSERT_TRUE(k1.stream().native_handle() == user_stream);
  ASSERT_TRUE(k0.get() == expect && k1.get() == expect);

  // a chain on one stream: sort, then scan into another vector, then reduce the scan's last run
  thrust::device_vector<int> sorted = h, scanned(n), slot(1);
  thrust::host_vector<int> hs = h, hscan(n);
  thrust::sort(hs.begin(), hs.end());
  thrust::inclusive_scan(hs.begin(), hs.end(), hscan.begin());
  auto e0 = thrust::async::sort(thrust::device.on(user_stream), sorted.begin(), sorted.end());
  auto e1 = thrust::async::inclusive_scan(thrust::device.after(e0), sorted.begin(), sorted.end(), scanned.begin());
  ASSERT_TRUE(e1.stream().native_handle() == user_stream);
  auto e2 = thrust::async::reduce_into(thrust::device.after(e1), sorted.begin(), sorted.end(), slot.begin(), 3, thrust::plus<int>());
  e2.wait();
  ASSERT_EQUAL_VEC(to_host(sorted), hs);
  ASSERT_EQUAL_VEC(to_host(scanned), hscan);
  ASSERT_TRUE((int)slot[0] == expect + 3);

  // work on another stream that depends on the chain: descending sort of the scan, exclusive scan, copy
  thrust::device_vector<int> desc(n), copied(n);
  auto c0 = thrust::async::copy(thrust::device.after(e1), scanned.begin(), scanned.end(), desc.begin());
  auto c1 = thrust::async::sort(thrust::device.after(c0), desc.begin(), desc.end(), thrust::greater<int>());
  auto c2 = thrust::async::exclusive_scan(thrust::device.after(c1), desc.begin(), desc.end(), copied.begin(), 11);
  thrust::when_all_wait(c2, e2);
  thrust::host_vector<int> hdesc = hscan, hex(n);
  thrust::sort(hdesc.begin(), hdesc.end(), thrust::greater<int>());
  thrust::exclusive_scan(hdesc.begin(), hdesc.end(), hex.begin(), 11);
  ASSERT_EQUAL_VEC(to_host(desc), hdesc);
  ASSERT_EQUAL_VEC(to_host(copied), hex);

  // host <-> device copies complete before they return; the event is ready
  thrust::device_vector<int> up(n);
  auto u0 = thrust::async::copy(h.begin(), h.end(), up.begin());
  ASSERT_EQUAL_VEC(to_host(up), h);
  u0.wait();

  // a synchronous algorithm accepts the same policies and waits for the dependencies itself
  auto s0 = thrust::async::reduce(d1.begin(), d1.end());
  ASSERT_TRUE(thrust::reduce(thrust::device.after(s0), d1.begin(), d1.end()) == expect);

  // with a caller's allocator: the temporary storage goes back when the future dies
  {
    CachingTempAllocator alloc;
    {
      auto a0 = thrust::async::reduce(thrust::device(alloc), d2.begin(), d2.end());
      ASSERT_TRUE(a0.get() == expect && alloc.live.size() == 1);
    }
    ASSERT_TRUE(alloc.live.empty() && alloc.returned == 1);
  }
  // empty range: the value is init
  auto z = thrust::async::reduce(d0.begin(), d0.begin(), 42);
  ASSERT_TRUE(z.get() == 42);
  k0 = thrust::device_future<int>();  // futures let go of the user's stream before it is destroyed
  k1 = thrust::device_future<int>();
  e0 = thrust::device_event(); e1 = thrust::device_event(); e2 = thrust::device_event();
  c0 = thrust::device_event(); c1 = thrust::device_event(); c2 = thrust::device_event();
  ASSERT_TRUE(thrust_amd_stream_synchronize(user_stream) == 0);
  ASSERT_TRUE(thrust_amd_stream_destroy(user_stream) == 0);
}

// Memory resources, allocators over them and allocator-aware device_vector (the reference:
// testing/mr_pool.cu, testing/allocator.cu, testing/caching_allocator.cu,
// examples/mr_basic.cu).
static void TestUniversalVector() {  // testing/universal_memory.cu:25-82: one pointer for host code and algorithms
  g_test = "UniversalVector";
  const size_t n = 100003;
  thrust::universal_vector<unsigned int> u(n);
  unsigned int* direct = thrust::raw_pointer_cast(u.data());
  thrust::host_vector<unsigned int> h(n);
  for (size_t i = 0; i < n; ++i) h[i] = direct[i] = (unsigned int)mix(i * 77 + 1);  // written by plain host stores
  thrust::sort(u.begin(), u.end());                                                 // sorted by the device system
  thrust::sort(h.begin(), h.end());
  bool ok = true;
  for (size_t i = 0; i < n; ++i) ok = ok && direct[i] == h[i];                      // read back by plain host loads
  ASSERT_TRUE(ok);
  ASSERT_TRUE(thrust::reduce(u.begin(), u.end(), 0u) == thrust::reduce(h.begin(), h.end(), 0u));
  ASSERT_TRUE(u[5] == h[5]);
  u[5] = 123u;
  ASSERT_TRUE(direct[5] == 123u);
  thrust::device_vector<unsigned int> d(u.begin(), u.end());  // universal -> device
  h[5] = 123u;
  ASSERT_EQUAL_VEC(to_host(d), h);
  thrust::universal_vector<unsigned int> scanned(n);
  thrust::inclusive_scan(d.begin(), d.end(), scanned.begin());  // device -> universal output
  thrust::host_vector<unsigned int> hs(n);
  thrust::inclusive_scan(h.begin(), h.end(), hs.begin());
  ok = true;
  const unsigned int* sdirect = thrust::raw_pointer_cast(scanned.data());
  for (size_t i = 0; i < n; ++i) ok = ok && sdirect[i] == hs[i];
  ASSERT_TRUE(ok);
  thrust::universal_vector<int> empty;
  ASSERT_TRUE(empty.size() == 0 && empty.begin() == empty.end());
}

// A block released on a stream that is destroyed afterwards must stay usable: the arena keeps
// an event per block, never the stream.  async::reduce runs on a stream of its own and gives
// its temporary storage back on that stream; dropping the future destroys the stream; the
// synchronous reduce of the same size on the null stream then picks that very block up.
// thrust/detail/vector_base.inl:165-180 in the reference: a host_vector built from a range of
// device iterators copies the range in one piece (here: a million elements in far less time
// than a million single reads would take), converting the elements if the types differ.
static void TestHostVectorFromDeviceRange() {
  g_test = "host_vector from a device range";
  const size_t n = 1u << 20;
  thrust::host_vector<int> src(n);
  for (size_t i = 0; i < n; ++i) src[i] = (int)i + 7;
  thrust::device_vector<int> d(src);
  thrust::host_vector<int> h(d.begin() + 5, d.end() - 3);
  ASSERT_TRUE(h.size() == n - 8);
  bool ok = true;
  for (size_t i = 0; i < h.size(); ++i) ok = ok && h[i] == (int)(i + 12);
  ASSERT_TRUE(ok);
  thrust::host_vector<long long> wide(d.begin(), d.begin() + 100);
  ASSERT_TRUE(wide.size() == 100 && wide[0] == 7 && wide[99] == 106);
  thrust::host_vector<int> none(d.begin(), d.begin());
  ASSERT_TRUE(none.empty());
}

static void TestTempArenaOutlivesStream() {
  g_test = "TempArenaOutlivesStream";
  ASSERT_TRUE(thrust_amd_temp_trim() == 0);  // nothing cached: the next block is the only one
  const size_t n = (1 << 20) + 3;
  thrust::host_vector<int> h = random_integers<int>(n, 11, 0);
  thrust::device_vector<int> d = h;
  long long total = 0;
  for (size_t i = 0; i < n; ++i) total += h[i];
  {
    auto f = thrust::async::reduce(d.begin(), d.end());
    ASSERT_TRUE(f.get() == (int)total);
  }  // the future, and with it its stream, is gone here
  const size_t held = thrust_amd_temp_bytes_held();
  ASSERT_TRUE(held > 0);
  int got = 0;
  bool threw = false;
  try {
    got = thrust::reduce(d.begin(), d.end());
  } catch (...) {
    threw = true;
  }
  ASSERT_TRUE(!threw);
  ASSERT_TRUE(got == (int)total);
  ASSERT_TRUE(thrust_amd_temp_bytes_held() == held);  // the cached block was reused, not lost
  // the same through the C ABI with a user's stream: release, destroy, acquire elsewhere
  void* s = nullptr;
  ASSERT_TRUE(thrust_amd_stream_create(&s) == 0);
  void* blk = nullptr;
  ASSERT_TRUE(thrust_amd_temp_acquire(&blk, 1 << 16, s) == 0 && blk != nullptr);
  ASSERT_TRUE(thrust_amd_temp_release(blk, s) == 0);
  ASSERT_TRUE(thrust_amd_stream_synchronize(s) == 0);
  ASSERT_TRUE(thrust_amd_stream_destroy(s) == 0);
  void* again = nullptr;
  ASSERT_TRUE(thrust_amd_temp_acquire(&again, 1 << 16, nullptr) == 0);
  ASSERT_TRUE(again == blk);
  ASSERT_TRUE(thrust_amd_temp_release(again, nullptr) == 0);
  ASSERT_TRUE(thrust_amd_temp_release(again, nullptr) != 0);  // not handed out any more
  ASSERT_TRUE(thrust_amd_temp_trim() == 0);
  ASSERT_TRUE(thrust_amd_temp_bytes_held() == 0);
}

// The other pool resources: the disjoint pool (bookkeeping in host memory, blocks carved from
// chunks), and the two mutex-guarded wrappers shared by several host threads
// (testing/mr_disjoint_pool.cu and testing/mr_pool.cu check the same behaviour: reuse of
// returned blocks, chunk growth, oversized blocks, release).
static void TestPoolResources() {
  g_test = "DisjointPool";
  typedef thrust::mr::disjoint_unsynchronized_pool_resource<thrust::device_memory_resource> Disjoint;
  thrust::device_memory_resource upstream;
  thrust::mr::new_delete_resource book;
  {
    Disjoint pool(&upstream, &book);
    // 16 blocks of 256 bytes per first chunk: 17 allocations take two chunks
    std::vector<thrust::device_ptr<void> > blocks;
    for (int i = 0; i < 17; ++i) blocks.push_back(pool.allocate(200));
    ASSERT_TRUE(pool.chunks() == 2 && pool.upstream_allocations() == 2);
    bool distinct = true, aligned = true;
    for (size_t i = 0; i < blocks.size(); ++i) {
      aligned = aligned && (reinterpret_cast<std::uintptr_t>(blocks[i].get()) % 256 == 0);
      for (size_t j = 0; j < i; ++j) distinct = distinct && blocks[i].get() != blocks[j].get();
    }
    ASSERT_TRUE(distinct && aligned);
    // a returned block is the next one handed out for its size
    pool.deallocate(blocks[5], 200);
    thrust::device_ptr<void> again = pool.allocate(256);
    ASSERT_TRUE(again.get() == blocks[5].get() && pool.upstream_allocations() == 2);
    // the blocks are device memory: fill one and read it back
    thrust::device_ptr<int> ints(static_cast<int*>(blocks[3].get()));
    thrust::fill(ints, ints + 50, 7);
    ASSERT_TRUE(thrust::reduce(ints, ints + 50) == 350);
    // oversized blocks are cached and reused for requests of a similar size
    thrust::device_ptr<void> big = pool.allocate((size_t)3 << 20);
    const size_t calls = pool.upstream_allocations();
    pool.deallocate(big, (size_t)3 << 20);
    ASSERT_TRUE(pool.cached_oversized_blocks() == 1);
    thrust::device_ptr<void> big2 = pool.allocate((size_t)2 << 20);
    ASSERT_TRUE(big2.get() == big.get() && pool.upstream_allocations() == calls);
    pool.deallocate(big2, (size_t)2 << 20);
    for (auto& b : blocks) pool.deallocate(b, 200);
    pool.release();
    ASSERT_TRUE(pool.chunks() == 0 && pool.cached_oversized_blocks() == 0);
    // vectors and temporary storage from the pool
    typedef thrust::mr::allocator<int, Disjoint> Alloc;
    Alloc alloc(&pool);
    thrust::host_vector<int> h = random_integers<int>(5000, 21, 0), hs = h;
    std::sort(hs.begin(), hs.end());
    {
      thrust::device_vector<int, Alloc> v(h.begin(), h.end(), alloc);
      thrust::sort(thrust::device(&pool), v.begin(), v.end());
      ASSERT_EQUAL_VEC(to_host(v), hs);
    }
    const size_t before = pool.upstream_allocations();
    {
      thrust::device_vector<int, Alloc> v(h.begin(), h.end(), alloc);
      thrust::sort(thrust::device(&pool), v.begin(), v.end());
      ASSERT_EQUAL_VEC(to_host(v), hs);
    }
    ASSERT_TRUE(pool.upstream_allocations() == before);  // everything came from the pool's chunks
  }
  g_test = "SynchronizedPools";
  {
    thrust::mr::synchronized_pool_resource<thrust::device_memory_resource> sync(&upstream);
    thrust::mr::disjoint_synchronized_pool_resource<thrust::device_memory_resource> dsync(&upstream, &book);
    std::atomic<int> bad(0);
    auto worker = [&](int id) {
      for (int round = 0; round < 200; ++round) {
        const size_t bytes = 256 + 64 * (size_t)((id * 7 + round) % 9);
        thrust::device_ptr<void> a = sync.allocate(bytes), b = dsync.allocate(bytes);
        if (!a.get() || !b.get() || a.get() == b.get()) ++bad;
        sync.deallocate(a, bytes);
        dsync.deallocate(b, bytes);
      }
    };
    std::thread t0(worker, 0), t1(worker, 1), t2(worker, 2), t3(worker, 3);
    t0.join(); t1.join(); t2.join(); t3.join();
    ASSERT_TRUE(bad.load() == 0);
    ASSERT_TRUE(sync.upstream_allocations() <= 4 * 4 && dsync.upstream_allocations() <= 8);
    sync.release();
    dsync.release();
  }
}

static void TestMemoryResources() {
  g_test = "MemoryResources";
  typedef thrust::mr::unsynchronized_pool_resource<thrust::device_memory_resource> Pool;
  thrust::device_memory_resource upstream;
  {
    Pool pool(&upstream);
    // the resource interface: blocks of a size class come back from the cache
    thrust::device_ptr<void> a = pool.allocate(1000);
    thrust::device_ptr<void> b = pool.allocate(1000);
    ASSERT_TRUE(a.get() != nullptr && b.get() != nullptr && a.get() != b.get());
    ASSERT_TRUE(pool.upstream_allocations() == 2);
    pool.deallocate(a, 1000);
    thrust::device_ptr<void> c = pool.allocate(900);  // same class (1024)
    ASSERT_TRUE(c.get() == a.get() && pool.upstream_allocations() == 2);
    pool.deallocate(b, 1000);
    pool.deallocate(c, 900);
    ASSERT_TRUE(pool.cached_bytes() == 2048);
    pool.release();
    ASSERT_TRUE(pool.cached_bytes() == 0);
    ASSERT_TRUE(pool == pool && !(pool != pool));

    // a vector over the pool: growing and shrinking reuses cached blocks
    typedef thrust::mr::allocator<int, Pool> PoolAlloc;
    PoolAlloc alloc(&pool);
    const std::size_t before = pool.upstream_allocations();
    {
      thrust::device_vector<int, PoolAlloc> v(1000, 7, alloc);
      ASSERT_TRUE(thrust::reduce(v.begin(), v.end()) == 7000);
      thrust::host_vector<int> h = random_integers<int>(1000, 9, 0);
      thrust::device_vector<int, PoolAlloc> w(alloc);
      w = thrust::device_vector<int, PoolAlloc>(h.begin(), h.end(), alloc);
      (void)w;
    }
    {
      thrust::device_vector<int, PoolAlloc> v(1000, 1, alloc);  // the block the first vector returned
      ASSERT_TRUE(pool.upstream_allocations() - before <= 2);
      thrust::host_vector<int> h = random_integers<int>(1000, 9, 0), hs = h;
      thrust::copy(h.begin(), h.end(), v.begin());
      thrust::sort(v.begin(), v.end());
      std::sort(hs.begin(), hs.end());
      ASSERT_EQUAL_VEC(to_host(v), hs);
      ASSERT_TRUE(v.get_allocator() == alloc);
      // vectors with different allocators compare and convert
      thrust::device_vector<int> plain(v);
      ASSERT_TRUE(plain == v);
    }
    // temporary storage of the algorithms from the pool: thrust::device(&pool)
    thrust::host_vector<int> h = random_integers<int>(1 << 16, 3, 0), hs = h;
    std::sort(hs.begin(), hs.end());
    thrust::device_vector<int> d = h;
    const std::size_t before_sort = pool.upstream_allocations();
    for (int round = 0; round < 3; ++round) {
      d = h;
      thrust::sort(thrust::device(&pool), d.begin(), d.end());
      ASSERT_EQUAL_VEC(to_host(d), hs);
    }
    ASSERT_TRUE(pool.upstream_allocations() - before_sort == 1);  // one new block, reused twice
    ASSERT_TRUE(thrust::reduce(thrust::hip::par(&pool).on(nullptr), d.begin(), d.end(), 0) ==
                thrust::reduce(d.begin(), d.end(), 0));
  }
  // the default allocator: stateless, all instances equal, usable directly
  thrust::device_allocator<int> da, db;
  ASSERT_TRUE(da == db);
  thrust::device_ptr<int> p = da.allocate(10);
  thrust::fill(p, p + 10, 3);
  ASSERT_TRUE(thrust::reduce(p, p + 10) == 30);
  da.deallocate(p, 10);
  thrust::device_vector<int> dv(5, 2);
  ASSERT_TRUE(dv.get_allocator() == da);
}

int main() {
  TestReduceSimple();
  TestReduceWithOperatorTable();
  TestScanSimple();
  TestMixedTypes();
  TestScanByKeySimple();
  TestCountSimple();
  TestInnerProductSimple();
  TestTransformReduceAndScanSimple();
  TestRemoveSimple();
  TestSetOperationsSimple();
  TestSortSimple();
  TestSortByKeySimple();
  TestReduceByKeySimple();
  TestUniqueSimple();
  TestUniqueByKeySimple();
  TestCopyIfSimple();
  TestStablePartitionSimple();
  TestMergeSimple();
  TestMergeByKeySimple();
  DifferentialForType<signed char>("signed char");
  DifferentialForType<short>("short");
  DifferentialForType<int>("int");
  DifferentialForType<unsigned int>("unsigned int");
  DifferentialForType<long long>("long long");
  DifferentialForType<unsigned long long>("unsigned long long");
  DifferentialForType<float>("float");
  DifferentialForType<double>("double");
  TestFloatSortTotalOrder();
  TestDispatch();
  TestPoliciesAndRawPointers();
  TestDeviceVector();
  TestOutOfMemoryThrows();
  TestMixedTypePlaceholders();
  TestRemoveIfKeepsNaN();
  TestTempArenaReuse();
  TestCustomTemporaryAllocation();
  TestAsyncAlgorithms();
  TestTempArenaOutlivesStream();
  TestMemoryResources();
  TestPoolResources();
  TestHostVectorFromDeviceRange();
  TestUniversalVector();
  std::printf("%s: %d checks, %d failed\n", g_failed ? "FAILED" : "PASSED", g_checks, g_failed);
  return g_failed ? 1 : 0;
}
