// Front-end test compiled with hipcc: more cases of the reference's own unit tests whose inputs
// or outputs are not plain arrays of numbers.
//   * sorts through a permutation iterator (testing/sort_permutation_iterator.cu:58-215),
//     keys and values of 4 to 1024 bytes (stable_sort_large.cu:6-44,
//     stable_sort_by_key_large_keys.cu, ..._large_values.cu), keys that use only their low
//     bits (sort_variable_bits.cu:20-50);
//   * scan_by_key with a predicate that reads head flags, a transform iterator as values,
//     key values that come back later, mixed value / output types, discard_iterator as
//     output, many sizes, values of 4 to 256 bytes (scan_by_key.cu:240-720);
//   * merge / merge_by_key into a discard_iterator and by thrust::greater
//     (merge.cu:143-204, merge_by_key.cu:198-318); set operations on equal ranges, on
//     multisets and into a discard_iterator (set_intersection.cu:150-260, set_union.cu,
//     set_difference.cu, set_symmetric_difference.cu);
//   * remove_copy(_if) into discard and zip iterators (remove.cu:520-800);
//   * transform scans from a struct to int, from a counting iterator, into a discard_iterator,
//     with thrust::identity<> / thrust::maximum<> (transform_scan.cu:195-401).
// Literal vectors are the reference's; everything else compares the device system with the
// sequential host system on the same inputs, and with the C++ standard library where it has
// the algorithm.
#include <thrust/copy.h>
#include <thrust/device_vector.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/iterator/constant_iterator.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/discard_iterator.h>
#include <thrust/iterator/permutation_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/merge.h>
#include <thrust/remove.h>
#include <thrust/scan.h>
#include <thrust/set_operations.h>
#include <thrust/sort.h>
#include <thrust/transform_scan.h>
#include <thrust/tuple.h>

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <iterator>
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
template <typename T>
static thrust::host_vector<T> hv(std::initializer_list<T> l) { return thrust::host_vector<T>(std::vector<T>(l)); }
template <typename T>
static thrust::host_vector<T> to_host(const thrust::device_vector<T>& d) { return thrust::host_vector<T>(d); }

static uint64_t mix(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
template <typename T>
static thrust::host_vector<T> random_integers(size_t n, uint64_t seed) {
  thrust::host_vector<T> h(n);
  for (size_t i = 0; i < n; ++i) h[i] = (T)mix(seed * 1000003ull + i);
  return h;
}
// keys 0, 0, 1, 1, 1, 2 ...: the key goes up after an element with probability 1 / every
template <typename K>
static thrust::host_vector<K> segment_keys(size_t n, uint64_t seed, unsigned every) {
  thrust::host_vector<K> h(n);
  size_t k = 0;
  for (size_t i = 0; i < n; ++i) {
    h[i] = (K)k;
    if (mix(seed * 7919ull + i) % every == 0) ++k;
  }
  return h;
}

static const size_t kSizes[] = {0, 1, 2, 63, 64, 65, 1000, 4097, 10027, 65539, (1u << 18) + 7};

// an element of N values of T, ordered by the first, added slot by slot
template <typename T, unsigned int N>
struct FixedVector {
  T data[N];
  __host__ __device__ FixedVector() {
    for (unsigned int i = 0; i < N; ++i) data[i] = T();
  }
  __host__ __device__ explicit FixedVector(T init) {
    for (unsigned int i = 0; i < N; ++i) data[i] = init;
  }
  __host__ __device__ FixedVector operator+(const FixedVector& o) const {
    FixedVector r;
    for (unsigned int i = 0; i < N; ++i) r.data[i] = data[i] + o.data[i];
    return r;
  }
  __host__ __device__ bool operator<(const FixedVector& o) const { return data[0] < o.data[0]; }
  __host__ __device__ bool operator==(const FixedVector& o) const {
    for (unsigned int i = 0; i < N; ++i)
      if (!(data[i] == o.data[i])) return false;
    return true;
  }
};

// ------------------------------------------------------------------ sorts through a permutation iterator
struct stride_functor {
  std::ptrdiff_t stride;
  __host__ __device__ std::ptrdiff_t operator()(const std::ptrdiff_t& i) const { return stride * i; }
};
template <typename Iterator>
struct strided_range {
  typedef thrust::counting_iterator<std::ptrdiff_t> CountingIterator;
  typedef thrust::transform_iterator<stride_functor, CountingIterator> TransformIterator;
  typedef thrust::permutation_iterator<Iterator, TransformIterator> iterator;
  Iterator first, last;
  std::ptrdiff_t stride;
  iterator begin() const { return iterator(first, TransformIterator(CountingIterator(0), stride_functor{stride})); }
  iterator end() const { return begin() + ((last - first) + (stride - 1)) / stride; }
};

template <typename Vector>
static void SortPermutationIterator() {
  typedef typename Vector::value_type T;
  typedef typename Vector::iterator Iterator;
  auto vec = [](std::initializer_list<T> l) { return Vector(thrust::host_vector<T>(std::vector<T>(l))); };
  for (int stable = 0; stable < 2; ++stable) {
    g_test = stable ? "StableSortPermutationIterator" : "SortPermutationIterator";
    Vector A = vec({2, 9, 0, 1, 5, 3, 8, 6, 7, 4});
    strided_range<Iterator> S{A.begin(), A.end(), 2};
    if (stable) thrust::stable_sort(S.begin(), S.end());
    else thrust::sort(S.begin(), S.end());
    ASSERT_TRUE(same(thrust::host_vector<T>(A), hv<T>({0, 9, 2, 1, 5, 3, 7, 6, 8, 4})));
    g_test = stable ? "StableSortByKeyPermutationIterator" : "SortByKeyPermutationIterator";
    Vector K = vec({2, 9, 0, 1, 5, 3, 8, 6, 7, 4}), V = vec({0, 1, 2, 3, 4, 5, 6, 7, 8, 9});
    strided_range<Iterator> SK{K.begin(), K.end(), 2}, SV{V.begin(), V.end(), 2};
    if (stable) thrust::stable_sort_by_key(SK.begin(), SK.end(), SV.begin());
    else thrust::sort_by_key(SK.begin(), SK.end(), SV.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(K), hv<T>({0, 9, 2, 1, 5, 3, 7, 6, 8, 4})));
    ASSERT_TRUE(same(thrust::host_vector<T>(V), hv<T>({2, 1, 0, 3, 4, 5, 8, 7, 6, 9})));
  }
}

static void TestSortPermutationIterators() {
  SortPermutationIterator<thrust::host_vector<int> >();
  SortPermutationIterator<thrust::device_vector<int> >();
  SortPermutationIterator<thrust::device_vector<short> >();
  SortPermutationIterator<thrust::device_vector<double> >();
  // every third element of a larger array; the others must stay where they are
  g_test = "SortPermutationIterator, large";
  const size_t n = 100003;
  thrust::host_vector<int> h = random_integers<int>(n, 11);
  thrust::device_vector<int> d = h;
  strided_range<thrust::device_vector<int>::iterator> S{d.begin(), d.end(), 3};
  thrust::sort(S.begin(), S.end());
  std::vector<int> every_third;
  for (size_t i = 0; i < n; i += 3) every_third.push_back(h[i]);
  std::sort(every_third.begin(), every_third.end());
  thrust::host_vector<int> got = d;
  bool ok = true;
  for (size_t i = 0; i < n; ++i) ok = ok && got[i] == (i % 3 == 0 ? every_third[i / 3] : h[i]);
  ASSERT_TRUE(ok);
}

// ------------------------------------------------------------------ large keys and values
template <unsigned int N>
static void StableSortWithLargeKeys() {
  typedef FixedVector<int, N> E;
  const size_t n = (128 * 1024) / sizeof(E);
  thrust::host_vector<E> h_keys(n);
  for (size_t i = 0; i < n; ++i) h_keys[i] = E((int)(mix(N * 131ull + i) % 1000));  // many ties
  thrust::device_vector<E> d_keys = h_keys;
  std::vector<E> expect(h_keys.begin(), h_keys.end());
  std::stable_sort(expect.begin(), expect.end());
  thrust::stable_sort(h_keys.begin(), h_keys.end());
  thrust::stable_sort(d_keys.begin(), d_keys.end());
  ASSERT_TRUE(same(h_keys, expect));
  ASSERT_TRUE(same(to_host(d_keys), expect));
}
template <unsigned int N>
static void StableSortByKeyWithLargeKeysAndValues() {
  typedef FixedVector<int, N> E;
  const size_t n = (128 * 1024) / sizeof(E);
  thrust::host_vector<E> h_keys(n);
  thrust::host_vector<unsigned int> h_vals(n);
  for (size_t i = 0; i < n; ++i) {
    h_keys[i] = E((int)(mix(N * 977ull + i) % 100));
    h_vals[i] = (unsigned int)i;
  }
  thrust::device_vector<E> d_keys = h_keys;
  thrust::device_vector<unsigned int> d_vals = h_vals;
  std::vector<unsigned int> order(n);
  for (size_t i = 0; i < n; ++i) order[i] = (unsigned int)i;
  std::stable_sort(order.begin(), order.end(), [&](unsigned a, unsigned b) { return h_keys[a] < h_keys[b]; });
  thrust::stable_sort_by_key(d_keys.begin(), d_keys.end(), d_vals.begin());
  ASSERT_TRUE(same(to_host(d_vals), order));
  // large values under small keys
  thrust::host_vector<unsigned int> h_small(n);
  thrust::host_vector<E> h_big(n);
  for (size_t i = 0; i < n; ++i) {
    h_small[i] = (unsigned int)(mix(N * 31ull + i) % 100);
    h_big[i] = E((int)i);
  }
  thrust::device_vector<unsigned int> d_small = h_small;
  thrust::device_vector<E> d_big = h_big;
  thrust::stable_sort_by_key(h_small.begin(), h_small.end(), h_big.begin());
  thrust::stable_sort_by_key(d_small.begin(), d_small.end(), d_big.begin());
  ASSERT_TRUE(same(to_host(d_small), h_small));
  ASSERT_TRUE(same(to_host(d_big), h_big));
}

template <typename T>
static void SortVariableBits(uint64_t seed) {
  for (size_t n : {(size_t)1000, (size_t)65539}) {
    for (size_t num_bits = 0; num_bits < 8 * sizeof(T); num_bits += 3) {
      thrust::host_vector<T> h_keys = random_integers<T>(n, seed + num_bits);
      const uint64_t mask = (1ull << num_bits) - 1;
      for (size_t i = 0; i < n; ++i) h_keys[i] = (T)(h_keys[i] & mask);
      std::vector<T> reference(h_keys.begin(), h_keys.end());
      thrust::device_vector<T> d_keys = h_keys;
      std::sort(reference.begin(), reference.end());
      thrust::sort(h_keys.begin(), h_keys.end());
      thrust::sort(d_keys.begin(), d_keys.end());
      ASSERT_TRUE(same(h_keys, reference));
      ASSERT_TRUE(same(to_host(d_keys), reference));
    }
  }
}

static void TestSortsOfLargeAndNarrowKeys() {
  g_test = "StableSortWithLargeKeys";
  StableSortWithLargeKeys<1>();
  StableSortWithLargeKeys<2>();
  StableSortWithLargeKeys<4>();
  StableSortWithLargeKeys<8>();
  StableSortWithLargeKeys<16>();
  StableSortWithLargeKeys<32>();
  StableSortWithLargeKeys<64>();
  StableSortWithLargeKeys<128>();
  StableSortWithLargeKeys<256>();
  g_test = "StableSortByKeyWithLargeKeys / Values";
  StableSortByKeyWithLargeKeysAndValues<1>();
  StableSortByKeyWithLargeKeysAndValues<4>();
  StableSortByKeyWithLargeKeysAndValues<16>();
  StableSortByKeyWithLargeKeysAndValues<64>();
  g_test = "SortVariableBits";
  SortVariableBits<uint8_t>(1);
  SortVariableBits<uint16_t>(2);
  SortVariableBits<uint32_t>(3);
  SortVariableBits<uint64_t>(4);
}

// ------------------------------------------------------------------ scan_by_key
struct head_flag_predicate {
  template <typename T>
  __host__ __device__ bool operator()(const T&, const T& b) { return b ? false : true; }
};

template <typename Vector>
static void ScanByKeyKnownAnswers() {
  typedef typename Vector::value_type T;
  auto vec = [](std::initializer_list<T> l) { return Vector(thrust::host_vector<T>(std::vector<T>(l))); };
  {
    g_test = "ScanByKeyHeadFlags";
    Vector keys = vec({0, 1, 0, 0, 1, 1, 0}), vals = vec({1, 2, 3, 4, 5, 6, 7}), output(7, 0);
    thrust::inclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin(), head_flag_predicate(), thrust::plus<T>());
    ASSERT_TRUE(same(thrust::host_vector<T>(output), hv<T>({1, 2, 5, 9, 5, 6, 13})));
    thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin(), T(10), head_flag_predicate(), thrust::plus<T>());
    ASSERT_TRUE(same(thrust::host_vector<T>(output), hv<T>({10, 10, 12, 15, 10, 10, 16})));
  }
  {
    g_test = "InclusiveScanByKeyTransformIterator";
    Vector keys = vec({0, 1, 1, 1, 2, 3, 3}), vals = vec({1, 2, 3, 4, 5, 6, 7}), output(7, 0);
    thrust::inclusive_scan_by_key(keys.begin(), keys.end(), thrust::make_transform_iterator(vals.begin(), thrust::negate<T>()),
                                  output.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(output), hv<T>({(T)-1, (T)-2, (T)-5, (T)-9, (T)-5, (T)-6, (T)-13})));
  }
  {
    g_test = "ScanByKeyReusedKeys";
    Vector keys = vec({0, 1, 1, 1, 0, 1, 1}), vals = vec({1, 2, 3, 4, 5, 6, 7}), output(7, 0);
    thrust::inclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(output), hv<T>({1, 2, 5, 9, 5, 6, 13})));
    thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin(), T(10));
    ASSERT_TRUE(same(thrust::host_vector<T>(output), hv<T>({10, 10, 12, 15, 10, 10, 16})));
  }
}

template <typename T>
static void ScanByKeyAgainstHost(uint64_t seed) {
  for (size_t n : kSizes) {
    thrust::host_vector<int> h_keys = segment_keys<int>(n, seed + n, 10);
    thrust::device_vector<int> d_keys = h_keys;
    thrust::host_vector<T> h_vals(n);
    for (size_t i = 0; i < n; ++i) h_vals[i] = (T)(i % 10);
    thrust::device_vector<T> d_vals = h_vals;
    thrust::host_vector<T> h_output(n), expect(n);
    thrust::device_vector<T> d_output(n);
    for (size_t i = 0; i < n; ++i) expect[i] = (i && h_keys[i] == h_keys[i - 1]) ? (T)(expect[i - 1] + h_vals[i]) : h_vals[i];
    g_test = "InclusiveScanByKey";
    thrust::inclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_output.begin());
    thrust::inclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_output.begin());
    ASSERT_TRUE(same(h_output, expect));
    ASSERT_TRUE(same(to_host(d_output), expect));
    g_test = "ExclusiveScanByKey";
    for (size_t i = 0; i < n; ++i) expect[i] = (i && h_keys[i] == h_keys[i - 1]) ? (T)(expect[i - 1] + h_vals[i - 1]) : (T)11;
    thrust::exclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_output.begin(), (T)11);
    thrust::exclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_output.begin(), (T)11);
    ASSERT_TRUE(same(h_output, expect));
    ASSERT_TRUE(same(to_host(d_output), expect));
    g_test = "ExclusiveScanByKeyInPlace";
    thrust::device_vector<T> d_inplace = d_vals;
    thrust::exclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_inplace.begin(), d_inplace.begin(), (T)11);
    ASSERT_TRUE(same(to_host(d_inplace), expect));
    g_test = "InclusiveScanByKeyInPlace";
    d_inplace = d_vals;
    thrust::inclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_inplace.begin(), d_inplace.begin());
    thrust::inclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_output.begin());
    ASSERT_TRUE(same(to_host(d_inplace), h_output));

    g_test = "ScanByKeyDiscardOutput";
    auto out = thrust::make_discard_iterator();
    thrust::exclusive_scan_by_key(d_keys.cbegin(), d_keys.cend(), d_vals.cbegin(), out);
    thrust::exclusive_scan_by_key(d_keys.cbegin(), d_keys.cend(), d_vals.cbegin(), out, T{});
    thrust::exclusive_scan_by_key(d_keys.cbegin(), d_keys.cend(), d_vals.cbegin(), out, T{}, thrust::equal_to<int>{});
    thrust::exclusive_scan_by_key(d_keys.cbegin(), d_keys.cend(), d_vals.cbegin(), out, T{}, thrust::equal_to<int>{},
                                  thrust::multiplies<T>{});
    thrust::inclusive_scan_by_key(d_keys.cbegin(), d_keys.cend(), d_vals.cbegin(), out);
    thrust::inclusive_scan_by_key(d_keys.cbegin(), d_keys.cend(), d_vals.cbegin(), out, thrust::equal_to<int>{});
    auto end = thrust::inclusive_scan_by_key(d_keys.cbegin(), d_keys.cend(), d_vals.cbegin(), out, thrust::equal_to<int>{},
                                             thrust::multiplies<T>{});
    ASSERT_TRUE(end == thrust::make_discard_iterator(n));
  }
}

static void TestScanByKeyMixedTypes() {
  g_test = "ScanByKeyMixedTypes";
  const size_t n = 113;
  thrust::host_vector<int> h_keys = segment_keys<int>(n, 5, 10);
  thrust::device_vector<int> d_keys = h_keys;
  thrust::host_vector<unsigned int> h_vals = random_integers<unsigned int>(n, 6);
  for (size_t i = 0; i < n; ++i) h_vals[i] %= 10;
  thrust::device_vector<unsigned int> d_vals = h_vals;
  thrust::host_vector<float> h_float_output(n);
  thrust::device_vector<float> d_float_output(n);
  thrust::host_vector<int> h_int_output(n);
  thrust::device_vector<int> d_int_output(n);
  thrust::inclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_float_output.begin());
  thrust::inclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_float_output.begin());
  ASSERT_TRUE(same(to_host(d_float_output), h_float_output));
  thrust::exclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_float_output.begin(), (float)3.5);
  thrust::exclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_float_output.begin(), (float)3.5);
  ASSERT_TRUE(same(to_host(d_float_output), h_float_output));
  ASSERT_TRUE(h_float_output[0] == 3.5f);
  thrust::exclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_float_output.begin(), (int)3);
  thrust::exclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_float_output.begin(), (int)3);
  ASSERT_TRUE(same(to_host(d_float_output), h_float_output));
  thrust::exclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_int_output.begin(), (int)3);
  thrust::exclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_int_output.begin(), (int)3);
  ASSERT_TRUE(same(to_host(d_int_output), h_int_output));
  thrust::exclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_int_output.begin(), (float)3.5);
  thrust::exclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_int_output.begin(), (float)3.5);
  ASSERT_TRUE(same(to_host(d_int_output), h_int_output));
}

static void TestScanByKeyLargeInput() {
  g_test = "ScanByKeyLargeInput";
  const unsigned int N = 1 << 20;
  thrust::host_vector<unsigned int> sizes = random_integers<unsigned int>(10, 21);
  thrust::host_vector<unsigned int> h_vals = random_integers<unsigned int>(N, 22);
  thrust::device_vector<unsigned int> d_vals = h_vals;
  thrust::host_vector<unsigned int> h_output(N, 0);
  thrust::device_vector<unsigned int> d_output(N, 0);
  for (size_t i = 0; i < sizes.size(); ++i) {
    const unsigned int n = sizes[i] % N;
    thrust::host_vector<unsigned int> h_keys = segment_keys<unsigned int>(n, 23 + i, 100);
    thrust::device_vector<unsigned int> d_keys = h_keys;
    thrust::inclusive_scan_by_key(h_keys.begin(), h_keys.begin() + n, h_vals.begin(), h_output.begin());
    thrust::inclusive_scan_by_key(d_keys.begin(), d_keys.begin() + n, d_vals.begin(), d_output.begin());
    ASSERT_TRUE(same(to_host(d_output), h_output));
  }
}

template <unsigned int N>
static void ScanByKeyWithLargeTypes() {
  typedef FixedVector<int, N> E;
  const size_t n = (64 * 1024) / sizeof(E);
  thrust::host_vector<unsigned int> h_keys = segment_keys<unsigned int>(n, N, 5);
  thrust::host_vector<E> h_vals(n), h_output(n);
  for (size_t i = 0; i < n; ++i) h_vals[i] = E((int)i);
  thrust::device_vector<unsigned int> d_keys = h_keys;
  thrust::device_vector<E> d_vals = h_vals, d_output(n);
  thrust::inclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_output.begin());
  thrust::inclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_output.begin());
  ASSERT_TRUE(same(to_host(d_output), h_output));
  thrust::exclusive_scan_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), h_output.begin(), E(0));
  thrust::exclusive_scan_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_output.begin(), E(0));
  ASSERT_TRUE(same(to_host(d_output), h_output));
}

static void TestScanByKey() {
  ScanByKeyKnownAnswers<thrust::host_vector<int> >();
  ScanByKeyKnownAnswers<thrust::device_vector<int> >();
  ScanByKeyKnownAnswers<thrust::device_vector<short> >();
  ScanByKeyKnownAnswers<thrust::device_vector<long long> >();
  ScanByKeyKnownAnswers<thrust::device_vector<float> >();
  ScanByKeyAgainstHost<int>(31);
  ScanByKeyAgainstHost<unsigned char>(32);
  ScanByKeyAgainstHost<long long>(33);
  TestScanByKeyMixedTypes();
  TestScanByKeyLargeInput();
  g_test = "ScanByKeyWithLargeTypes";
  ScanByKeyWithLargeTypes<1>();
  ScanByKeyWithLargeTypes<2>();
  ScanByKeyWithLargeTypes<4>();
  ScanByKeyWithLargeTypes<8>();
  ScanByKeyWithLargeTypes<64>();
}

// ------------------------------------------------------------------ merge and set operations
template <typename T>
static void MergesAndSets(uint64_t seed) {
  for (size_t n : kSizes) {
    thrust::host_vector<T> h_a = random_integers<T>(n, seed + n), h_b = random_integers<T>(n, seed + 1000 + n);
    thrust::stable_sort(h_a.begin(), h_a.end());
    thrust::stable_sort(h_b.begin(), h_b.end());
    thrust::device_vector<T> d_a = h_a, d_b = h_b;

    g_test = "MergeToDiscardIterator";
    thrust::discard_iterator<> reference(2 * n);
    ASSERT_TRUE(thrust::merge(h_a.begin(), h_a.end(), h_b.begin(), h_b.end(), thrust::make_discard_iterator()) == reference);
    ASSERT_TRUE(thrust::merge(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), thrust::make_discard_iterator()) == reference);

    g_test = "MergeByKeyToDiscardIterator";
    {
      thrust::host_vector<T> h_av = random_integers<T>(n, seed + 3), h_bv = random_integers<T>(n, seed + 4);
      thrust::device_vector<T> d_av = h_av, d_bv = h_bv;
      thrust::host_vector<T> h_vals(2 * n), expect_keys(2 * n);
      thrust::device_vector<T> d_vals(2 * n), d_keys_out(2 * n);
      auto h_end = thrust::merge_by_key(h_a.begin(), h_a.end(), h_b.begin(), h_b.end(), h_av.begin(), h_bv.begin(),
                                        thrust::make_discard_iterator(), h_vals.begin());
      auto d_end = thrust::merge_by_key(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), d_av.begin(), d_bv.begin(),
                                        thrust::make_discard_iterator(), d_vals.begin());
      ASSERT_TRUE(h_end.first == reference && d_end.first == reference);
      ASSERT_TRUE(h_end.second == h_vals.end() && d_end.second == d_vals.end());
      ASSERT_TRUE(same(to_host(d_vals), h_vals));
      auto d_end2 = thrust::merge_by_key(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), d_av.begin(), d_bv.begin(),
                                         d_keys_out.begin(), thrust::make_discard_iterator());
      ASSERT_TRUE(d_end2.first == d_keys_out.end() && d_end2.second == reference);
      std::merge(h_a.begin(), h_a.end(), h_b.begin(), h_b.end(), expect_keys.begin());
      ASSERT_TRUE(same(to_host(d_keys_out), expect_keys));
    }

    g_test = "set operations: EquivalentRanges / ToDiscardIterator";
    {
      thrust::device_vector<T> d_same = d_a, d_result(2 * n);
      std::vector<T> expect(2 * n);
      auto check = [&](auto device_end, auto expect_end) {
        const size_t count = (size_t)(expect_end - expect.begin());
        ASSERT_TRUE((size_t)(device_end - d_result.begin()) == count);
        thrust::host_vector<T> got(d_result.begin(), d_result.begin() + count);
        ASSERT_TRUE(same(got, std::vector<T>(expect.begin(), expect.begin() + count)));
        return count;
      };
      // a range against itself
      check(thrust::set_intersection(d_a.begin(), d_a.end(), d_same.begin(), d_same.end(), d_result.begin()),
            std::set_intersection(h_a.begin(), h_a.end(), h_a.begin(), h_a.end(), expect.begin()));
      check(thrust::set_union(d_a.begin(), d_a.end(), d_same.begin(), d_same.end(), d_result.begin()),
            std::set_union(h_a.begin(), h_a.end(), h_a.begin(), h_a.end(), expect.begin()));
      check(thrust::set_difference(d_a.begin(), d_a.end(), d_same.begin(), d_same.end(), d_result.begin()),
            std::set_difference(h_a.begin(), h_a.end(), h_a.begin(), h_a.end(), expect.begin()));
      check(thrust::set_symmetric_difference(d_a.begin(), d_a.end(), d_same.begin(), d_same.end(), d_result.begin()),
            std::set_symmetric_difference(h_a.begin(), h_a.end(), h_a.begin(), h_a.end(), expect.begin()));
      // two ranges, into memory and into a discard_iterator
      const size_t n_int = check(thrust::set_intersection(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), d_result.begin()),
                                 std::set_intersection(h_a.begin(), h_a.end(), h_b.begin(), h_b.end(), expect.begin()));
      const size_t n_uni = check(thrust::set_union(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), d_result.begin()),
                                 std::set_union(h_a.begin(), h_a.end(), h_b.begin(), h_b.end(), expect.begin()));
      const size_t n_dif = check(thrust::set_difference(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), d_result.begin()),
                                 std::set_difference(h_a.begin(), h_a.end(), h_b.begin(), h_b.end(), expect.begin()));
      const size_t n_sym = check(
          thrust::set_symmetric_difference(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), d_result.begin()),
          std::set_symmetric_difference(h_a.begin(), h_a.end(), h_b.begin(), h_b.end(), expect.begin()));
      auto sink = thrust::make_discard_iterator();
      ASSERT_TRUE(thrust::set_intersection(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), sink) == thrust::make_discard_iterator(n_int));
      ASSERT_TRUE(thrust::set_union(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), sink) == thrust::make_discard_iterator(n_uni));
      ASSERT_TRUE(thrust::set_difference(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), sink) == thrust::make_discard_iterator(n_dif));
      ASSERT_TRUE(thrust::set_symmetric_difference(d_a.begin(), d_a.end(), d_b.begin(), d_b.end(), sink) == thrust::make_discard_iterator(n_sym));
      ASSERT_TRUE(thrust::set_union(h_a.begin(), h_a.end(), h_b.begin(), h_b.end(), sink) == thrust::make_discard_iterator(n_uni));
    }

    g_test = "set operations: Multiset";
    {
      // elements restricted to a few values, so that every value occurs many times on both sides
      thrust::host_vector<T> m_a(n), m_b(n);
      for (size_t i = 0; i < n; ++i) {
        m_a[i] = (T)((int)(mix(seed + 5 + i) % 25) - 12 < 0 && !std::is_signed<T>::value ? 0 : (int)(mix(seed + 5 + i) % 25) - 12);
        m_b[i] = (T)(int)(mix(seed + 6 + i) % 13);
      }
      std::sort(m_a.begin(), m_a.end());
      std::sort(m_b.begin(), m_b.end());
      thrust::device_vector<T> dm_a = m_a, dm_b = m_b, d_result(2 * n);
      std::vector<T> expect(2 * n);
      auto check = [&](auto device_end, auto expect_end) {
        const size_t count = (size_t)(expect_end - expect.begin());
        ASSERT_TRUE((size_t)(device_end - d_result.begin()) == count);
        thrust::host_vector<T> got(d_result.begin(), d_result.begin() + count);
        ASSERT_TRUE(same(got, std::vector<T>(expect.begin(), expect.begin() + count)));
      };
      check(thrust::set_intersection(dm_a.begin(), dm_a.end(), dm_b.begin(), dm_b.end(), d_result.begin()),
            std::set_intersection(m_a.begin(), m_a.end(), m_b.begin(), m_b.end(), expect.begin()));
      check(thrust::set_union(dm_a.begin(), dm_a.end(), dm_b.begin(), dm_b.end(), d_result.begin()),
            std::set_union(m_a.begin(), m_a.end(), m_b.begin(), m_b.end(), expect.begin()));
      check(thrust::set_difference(dm_a.begin(), dm_a.end(), dm_b.begin(), dm_b.end(), d_result.begin()),
            std::set_difference(m_a.begin(), m_a.end(), m_b.begin(), m_b.end(), expect.begin()));
      check(thrust::set_symmetric_difference(dm_a.begin(), dm_a.end(), dm_b.begin(), dm_b.end(), d_result.begin()),
            std::set_symmetric_difference(m_a.begin(), m_a.end(), m_b.begin(), m_b.end(), expect.begin()));
    }

    g_test = "MergeDescending";
    {
      thrust::host_vector<T> g_a = h_a, g_b = h_b;
      thrust::stable_sort(g_a.begin(), g_a.end(), thrust::greater<T>());
      thrust::stable_sort(g_b.begin(), g_b.end(), thrust::greater<T>());
      thrust::device_vector<T> dg_a = g_a, dg_b = g_b, d_result(2 * n);
      thrust::host_vector<T> h_result(2 * n);
      std::vector<T> expect(2 * n);
      std::merge(g_a.begin(), g_a.end(), g_b.begin(), g_b.end(), expect.begin(), std::greater<T>());
      auto h_end = thrust::merge(g_a.begin(), g_a.end(), g_b.begin(), g_b.end(), h_result.begin(), thrust::greater<T>());
      auto d_end = thrust::merge(dg_a.begin(), dg_a.end(), dg_b.begin(), dg_b.end(), d_result.begin(), thrust::greater<T>());
      ASSERT_TRUE(h_end == h_result.end() && d_end == d_result.end());
      ASSERT_TRUE(same(h_result, expect));
      ASSERT_TRUE(same(to_host(d_result), expect));
      // by key, descending: values follow their keys, ties from the first range first
      thrust::host_vector<int> va(n), vb(n), h_vals(2 * n);
      for (size_t i = 0; i < n; ++i) { va[i] = (int)i; vb[i] = (int)(n + i); }
      thrust::device_vector<int> dva = va, dvb = vb, d_vals(2 * n);
      thrust::merge_by_key(g_a.begin(), g_a.end(), g_b.begin(), g_b.end(), va.begin(), vb.begin(), h_result.begin(),
                           h_vals.begin(), thrust::greater<T>());
      thrust::merge_by_key(dg_a.begin(), dg_a.end(), dg_b.begin(), dg_b.end(), dva.begin(), dvb.begin(), d_result.begin(),
                           d_vals.begin(), thrust::greater<T>());
      ASSERT_TRUE(same(h_result, expect));
      ASSERT_TRUE(same(to_host(d_result), expect));
      ASSERT_TRUE(same(to_host(d_vals), h_vals));
    }
  }
}

static void TestMergesAndSetOperations() {
  MergesAndSets<int>(41);
  MergesAndSets<unsigned short>(42);
  MergesAndSets<long long>(43);
}

// ------------------------------------------------------------------ remove_copy into discard / zip outputs
template <typename T>
struct is_even {
  __host__ __device__ bool operator()(T x) { return (x & 1) == 0; }
};
template <typename T>
struct is_true {
  __host__ __device__ bool operator()(T x) { return x ? true : false; }
};

template <typename T>
static void RemoveCopyToDiscard(uint64_t seed) {
  for (size_t n : kSizes) {
    thrust::host_vector<T> h_data = random_integers<T>(n, seed + n);
    for (size_t i = 0; i < n; ++i) h_data[i] = (T)(h_data[i] % 4);
    thrust::device_vector<T> d_data = h_data;
    thrust::host_vector<T> h_stencil = random_integers<T>(n, seed + 50 + n);
    thrust::device_vector<T> d_stencil = h_stencil;

    g_test = "RemoveCopyToDiscardIterator";
    const size_t zeros = (size_t)std::count(h_data.begin(), h_data.end(), (T)0);
    thrust::discard_iterator<> reference(n - zeros);
    ASSERT_TRUE(thrust::remove_copy(h_data.begin(), h_data.end(), thrust::make_discard_iterator(), (T)0) == reference);
    ASSERT_TRUE(thrust::remove_copy(d_data.begin(), d_data.end(), thrust::make_discard_iterator(), (T)0) == reference);

    g_test = "RemoveCopyToDiscardIteratorZipped";
    {
      thrust::host_vector<T> h_output(n);
      thrust::device_vector<T> d_output(n);
      auto h_end = thrust::remove_copy(thrust::make_zip_iterator(thrust::make_tuple(h_data.begin(), h_data.begin())),
                                       thrust::make_zip_iterator(thrust::make_tuple(h_data.end(), h_data.end())),
                                       thrust::make_zip_iterator(thrust::make_tuple(h_output.begin(), thrust::make_discard_iterator())),
                                       thrust::make_tuple((T)0, (T)0));
      auto d_end = thrust::remove_copy(thrust::make_zip_iterator(thrust::make_tuple(d_data.begin(), d_data.begin())),
                                       thrust::make_zip_iterator(thrust::make_tuple(d_data.end(), d_data.end())),
                                       thrust::make_zip_iterator(thrust::make_tuple(d_output.begin(), thrust::make_discard_iterator())),
                                       thrust::make_tuple((T)0, (T)0));
      ASSERT_TRUE(thrust::get<0>(h_end.get_iterator_tuple()) == h_output.begin() + (n - zeros));
      ASSERT_TRUE(thrust::get<0>(d_end.get_iterator_tuple()) == d_output.begin() + (n - zeros));
      ASSERT_TRUE(thrust::get<1>(h_end.get_iterator_tuple()) == reference);
      ASSERT_TRUE(thrust::get<1>(d_end.get_iterator_tuple()) == reference);
      h_output.resize(n - zeros);
      d_output.resize(n - zeros);
      std::vector<T> expect;
      for (size_t i = 0; i < n; ++i)
        if (h_data[i] != (T)0) expect.push_back(h_data[i]);
      ASSERT_TRUE(same(h_output, expect));
      ASSERT_TRUE(same(to_host(d_output), expect));
    }

    g_test = "RemoveCopyIfToDiscardIterator";
    const size_t num_true = (size_t)std::count_if(h_data.begin(), h_data.end(), is_true<T>());
    ASSERT_TRUE(thrust::remove_copy_if(h_data.begin(), h_data.end(), thrust::make_discard_iterator(), is_true<T>()) ==
                thrust::make_discard_iterator(n - num_true));
    ASSERT_TRUE(thrust::remove_copy_if(d_data.begin(), d_data.end(), thrust::make_discard_iterator(), is_true<T>()) ==
                thrust::make_discard_iterator(n - num_true));

    g_test = "RemoveCopyIfStencilToDiscardIterator";
    const size_t num_even = (size_t)std::count_if(h_stencil.begin(), h_stencil.end(), is_even<T>());
    ASSERT_TRUE(thrust::remove_copy_if(h_data.begin(), h_data.end(), h_stencil.begin(), thrust::make_discard_iterator(),
                                       is_even<T>()) == thrust::make_discard_iterator(n - num_even));
    ASSERT_TRUE(thrust::remove_copy_if(d_data.begin(), d_data.end(), d_stencil.begin(), thrust::make_discard_iterator(),
                                       is_even<T>()) == thrust::make_discard_iterator(n - num_even));
  }
}

static void TestRemoveCopyOutputs() {
  RemoveCopyToDiscard<int>(51);
  RemoveCopyToDiscard<unsigned char>(52);
  RemoveCopyToDiscard<long long>(53);
}

// ------------------------------------------------------------------ transform scans
struct Record {
  int number;
  bool operator==(const Record& rhs) const { return number == rhs.number; }
};
struct negate_record {
  __host__ __device__ int operator()(Record const& record) const { return -record.number; }
};

static void TestTransformScans() {
  g_test = "TransformInclusiveScanDifferentTypes";
  {
    thrust::host_vector<Record> h_input(5);
    const int numbers[5] = {1, 3, -2, 4, -5};
    for (int i = 0; i < 5; ++i) h_input[i].number = numbers[i];
    thrust::host_vector<Record> input_copy(h_input);
    thrust::host_vector<int> h_output(5);
    auto h_iter = thrust::transform_inclusive_scan(h_input.begin(), h_input.end(), h_output.begin(), negate_record{}, thrust::plus<int>{});
    ASSERT_TRUE((size_t)(h_iter - h_output.begin()) == h_input.size());
    ASSERT_TRUE(same(h_input, input_copy));
    ASSERT_TRUE(same(h_output, hv<int>({-1, -4, -2, -6, -1})));
    thrust::device_vector<Record> d_input = h_input;
    thrust::device_vector<int> d_output(5);
    auto d_iter = thrust::transform_inclusive_scan(d_input.begin(), d_input.end(), d_output.begin(), negate_record{}, thrust::plus<int>{});
    ASSERT_TRUE((size_t)(d_iter - d_output.begin()) == d_input.size());
    ASSERT_TRUE(same(to_host(d_input), input_copy));
    ASSERT_TRUE(same(to_host(d_output), hv<int>({-1, -4, -2, -6, -1})));
  }
  g_test = "TransformScanCountingIterator";
  {
    thrust::counting_iterator<int> first(1);
    thrust::device_vector<int> result(3);
    thrust::transform_inclusive_scan(first, first + 3, result.begin(), thrust::negate<int>(), thrust::plus<int>());
    ASSERT_TRUE(same(to_host(result), hv<int>({-1, -3, -6})));
    thrust::transform_exclusive_scan(first, first + 3, result.begin(), thrust::negate<int>(), 0, thrust::plus<int>());
    ASSERT_TRUE(same(to_host(result), hv<int>({0, -1, -3})));
  }
  g_test = "TransformScanToDiscardIterator";
  for (size_t n : kSizes) {
    thrust::host_vector<int> h_input = random_integers<int>(n, 61 + n);
    thrust::device_vector<int> d_input = h_input;
    thrust::discard_iterator<> reference(n);
    ASSERT_TRUE(thrust::transform_inclusive_scan(h_input.begin(), h_input.end(), thrust::make_discard_iterator(),
                                                 thrust::negate<int>(), thrust::plus<int>()) == reference);
    ASSERT_TRUE(thrust::transform_inclusive_scan(d_input.begin(), d_input.end(), thrust::make_discard_iterator(),
                                                 thrust::negate<int>(), thrust::plus<int>()) == reference);
    ASSERT_TRUE(thrust::transform_exclusive_scan(h_input.begin(), h_input.end(), thrust::make_discard_iterator(),
                                                 thrust::negate<int>(), 0, thrust::plus<int>()) == reference);
    ASSERT_TRUE(thrust::transform_exclusive_scan(d_input.begin(), d_input.end(), thrust::make_discard_iterator(),
                                                 thrust::negate<int>(), 0, thrust::plus<int>()) == reference);
  }
}

template <typename T>
static void ValueCategoryDeduction() {
  g_test = "ValueCategoryDeduction";
  thrust::device_vector<T> vec;
  T a_h[10] = {5, 0, 5, 8, 6, 7, 5, 3, 0, 9};
  vec.assign((T*)a_h, a_h + 10);
  thrust::transform_inclusive_scan(thrust::device, vec.cbegin(), vec.cend(), vec.begin(), thrust::identity<>{},
                                   thrust::maximum<>{});
  ASSERT_TRUE(same(to_host(vec), hv<T>({5, 5, 5, 8, 8, 8, 8, 8, 8, 9})));
  vec.assign((T*)a_h, a_h + 10);
  thrust::transform_exclusive_scan(thrust::device, vec.cbegin(), vec.cend(), vec.begin(), thrust::identity<>{}, T{},
                                   thrust::maximum<>{});
  ASSERT_TRUE(same(to_host(vec), hv<T>({0, 5, 5, 5, 8, 8, 8, 8, 8, 8})));
}

int main() {
  TestSortPermutationIterators();
  TestSortsOfLargeAndNarrowKeys();
  TestScanByKey();
  TestMergesAndSetOperations();
  TestRemoveCopyOutputs();
  TestTransformScans();
  ValueCategoryDeduction<int>();
  ValueCategoryDeduction<unsigned char>();
  ValueCategoryDeduction<long long>();
  ValueCategoryDeduction<float>();
  ValueCategoryDeduction<double>();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
