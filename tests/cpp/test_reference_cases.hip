// Front-end test compiled with hipcc: cases of the reference's own unit tests for the hot-path
// algorithms that take forms of input or output the other programs here do not:
//   * bool keys (testing/sort.cu:107-134, sort_by_key.cu:100-140),
//   * std::vector / std::list / const iterators and std::vector<bool> as sources of thrust::copy
//     (testing/copy.cu:17-47, 167-224), mixed element types (copy.cu:108-163),
//   * discard_iterator as one or both outputs of copy, reduce_by_key, unique_copy,
//     unique_by_key_copy, partition_copy, stable_partition_copy and the scans
//     (copy.cu:49-106, reduce_by_key.cu:159-199, unique.cu:241-266, unique_by_key.cu:341-437,
//     partition.cu:474-975, scan.cu:264-330),
//   * predicates that return something other than bool, on random data and on a sequence
//     (copy.cu:289-371), random stencils (copy.cu:395-420), a type whose assignment needs
//     constructed memory (copy.cu:422-520),
//   * zip iterators as the range or the stencil of partition / stable_partition
//     (partition.cu:979-1160) and as the output of copy (copy.cu:541-579),
//   * operators that read a table through a pointer (reduce.cu:151-192, scan.cu:515-562),
//   * element types of 4, 32 and 256 bytes with their own operator+ under the default plus
//     (scan.cu:474-512, 656-675).
// Literal vectors are the reference's; everything else compares the device system with the
// sequential host system on the same inputs, and with a plain loop where one is at hand.
#include <thrust/copy.h>
#include <thrust/count.h>
#include <thrust/device_vector.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/iterator/constant_iterator.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/discard_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/partition.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/sequence.h>
#include <thrust/sort.h>
#include <thrust/tuple.h>
#include <thrust/unique.h>

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <iterator>
#include <list>
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
// random integers over the whole range of T, as unittest::random_integers<T> makes them
template <typename T>
static thrust::host_vector<T> random_integers(size_t n, uint64_t seed) {
  thrust::host_vector<T> h(n);
  for (size_t i = 0; i < n; ++i) h[i] = (T)mix(seed * 1000003ull + i);
  return h;
}
template <typename T>
static thrust::host_vector<T> random_bools(size_t n, uint64_t seed) {
  thrust::host_vector<T> h(n);
  for (size_t i = 0; i < n; ++i) h[i] = (T)(mix(seed * 1000003ull + i) & 1);
  return h;
}

static const size_t kSizes[] = {0, 1, 2, 63, 64, 65, 1000, 4097, 10027, 65539, (1u << 18) + 7};

// ------------------------------------------------------------------ bool keys
static void TestSortBool() {
  g_test = "SortBool";
  const size_t n = 10027;
  for (int descending = 0; descending < 2; ++descending) {
    thrust::host_vector<bool> h = random_bools<bool>(n, 1 + descending);
    thrust::device_vector<bool> d = h;
    if (descending) {
      thrust::sort(h.begin(), h.end(), thrust::greater<bool>());
      thrust::sort(d.begin(), d.end(), thrust::greater<bool>());
    } else {
      thrust::sort(h.begin(), h.end());
      thrust::sort(d.begin(), d.end());
    }
    ASSERT_TRUE(same(to_host(d), h));
    const size_t trues = (size_t)std::count(h.begin(), h.end(), true);
    // all of one value first, then all of the other
    bool ordered = true;
    for (size_t i = 0; i < n; ++i) ordered = ordered && (h[i] == (descending ? i < trues : i >= n - trues));
    ASSERT_TRUE(ordered);
  }
}

static void TestSortByKeyBool() {
  g_test = "SortByKeyBool";
  const size_t n = 10027;
  for (int descending = 0; descending < 2; ++descending) {
    thrust::host_vector<bool> hk = random_bools<bool>(n, 3 + descending);
    thrust::host_vector<int> hvals = random_integers<int>(n, 5 + descending);
    thrust::device_vector<bool> dk = hk;
    thrust::device_vector<int> dv = hvals;
    // the expected order by a stable partition of the indices
    std::vector<int> expect;
    for (int pass = 0; pass < 2; ++pass)
      for (size_t i = 0; i < n; ++i)
        if ((bool)hk[i] == (descending ? pass == 0 : pass == 1)) expect.push_back(hvals[i]);
    if (descending) {
      thrust::sort_by_key(hk.begin(), hk.end(), hvals.begin(), thrust::greater<bool>());
      thrust::sort_by_key(dk.begin(), dk.end(), dv.begin(), thrust::greater<bool>());
    } else {
      thrust::sort_by_key(hk.begin(), hk.end(), hvals.begin());
      thrust::sort_by_key(dk.begin(), dk.end(), dv.begin());
    }
    ASSERT_TRUE(same(to_host(dk), hk));
    ASSERT_TRUE(same(to_host(dv), hvals));
    ASSERT_TRUE(same(hvals, expect));  // both sorts are stable, so the values are pinned too
  }
}

// ------------------------------------------------------------------ thrust::copy from and to standard containers
template <typename Vector>
static void CopyFromStandardContainers() {
  typedef typename Vector::value_type T;
  {
    std::vector<T> v = {0, 1, 2, 3, 4};
    typename std::vector<T>::const_iterator begin = v.begin(), end = v.end();
    Vector d(5, (T)10);
    typename Vector::iterator r = thrust::copy(begin, end, d.begin());
    ASSERT_TRUE(r == d.end());
    for (int i = 0; i < 5; ++i) ASSERT_TRUE(d[i] == (T)i);
  }
  {
    std::list<T> l = {0, 1, 2, 3, 4};
    Vector v(l.size());
    typename Vector::iterator r = thrust::copy(l.begin(), l.end(), v.begin());
    ASSERT_TRUE(r == v.end());
    for (int i = 0; i < 5; ++i) ASSERT_TRUE(v[i] == (T)i);
    l.clear();
    thrust::copy(v.begin(), v.end(), std::back_insert_iterator<std::list<T> >(l));
    ASSERT_TRUE(l.size() == 5);
    int i = 0;
    for (T x : l) ASSERT_TRUE(x == (T)(i++));
  }
  {
    // to another element type
    Vector v(5);
    for (int i = 0; i < 5; ++i) v[i] = (T)i;
    thrust::host_vector<float> h(5, 10.0f);
    thrust::device_vector<float> d(5, 10.0f);
    ASSERT_TRUE(thrust::copy(v.begin(), v.end(), h.begin()) == h.end());
    ASSERT_TRUE(thrust::copy(v.begin(), v.end(), d.begin()) == d.end());
    for (int i = 0; i < 5; ++i) ASSERT_TRUE(h[i] == (float)i && d[i] == (float)i);
    // and the same type
    thrust::host_vector<T> h2(5, (T)10);
    thrust::device_vector<T> d2(5, (T)10);
    ASSERT_TRUE(thrust::copy(v.begin(), v.end(), h2.begin()) == h2.end());
    ASSERT_TRUE(thrust::copy(v.begin(), v.end(), d2.begin()) == d2.end());
    for (int i = 0; i < 5; ++i) ASSERT_TRUE(h2[i] == (T)i && d2[i] == (T)i);
  }
}

static void TestCopyStandardContainers() {
  g_test = "CopyStandardContainers";
  CopyFromStandardContainers<thrust::host_vector<int> >();
  CopyFromStandardContainers<thrust::device_vector<int> >();
  CopyFromStandardContainers<thrust::device_vector<short> >();
  CopyFromStandardContainers<thrust::device_vector<unsigned long long> >();
  g_test = "CopyVectorBool";
  std::vector<bool> v(3);
  v[0] = true; v[1] = false; v[2] = true;
  thrust::host_vector<bool> h(3);
  thrust::device_vector<bool> d(3);
  thrust::copy(v.begin(), v.end(), h.begin());
  thrust::copy(v.begin(), v.end(), d.begin());
  ASSERT_TRUE(h[0] == true && h[1] == false && h[2] == true);
  ASSERT_TRUE(d[0] == true && d[1] == false && d[2] == true);
}

static void TestCopyToDiscardAndZip() {
  g_test = "CopyToDiscardIterator";
  thrust::host_vector<int> h_input(5, 1);
  thrust::device_vector<int> d_input = h_input;
  thrust::discard_iterator<> reference(5);
  thrust::discard_iterator<> h_result = thrust::copy(h_input.begin(), h_input.end(), thrust::make_discard_iterator());
  thrust::discard_iterator<> d_result = thrust::copy(d_input.begin(), d_input.end(), thrust::make_discard_iterator());
  ASSERT_TRUE(reference == h_result);
  ASSERT_TRUE(reference == d_result);

  g_test = "CopyToDiscardIteratorZipped";
  {
    thrust::host_vector<int> h_output(5);
    thrust::device_vector<int> d_output(5);
    auto h_end = thrust::copy(thrust::make_zip_iterator(thrust::make_tuple(h_input.begin(), h_input.begin())),
                              thrust::make_zip_iterator(thrust::make_tuple(h_input.end(), h_input.end())),
                              thrust::make_zip_iterator(thrust::make_tuple(thrust::make_discard_iterator(), h_output.begin())));
    auto d_end = thrust::copy(thrust::make_zip_iterator(thrust::make_tuple(d_input.begin(), d_input.begin())),
                              thrust::make_zip_iterator(thrust::make_tuple(d_input.end(), d_input.end())),
                              thrust::make_zip_iterator(thrust::make_tuple(thrust::make_discard_iterator(), d_output.begin())));
    ASSERT_TRUE(same(h_output, h_input));
    ASSERT_TRUE(same(to_host(d_output), h_input));
    ASSERT_TRUE(reference == thrust::get<0>(h_end.get_iterator_tuple()));
    ASSERT_TRUE(reference == thrust::get<0>(d_end.get_iterator_tuple()));
  }

  g_test = "CopyCountingIterator";
  {
    thrust::counting_iterator<int> iter(1);
    thrust::device_vector<int> vec(4);
    thrust::copy(iter, iter + 4, vec.begin());
    ASSERT_TRUE(same(to_host(vec), hv<int>({1, 2, 3, 4})));
    thrust::host_vector<short> hvec(4);
    thrust::counting_iterator<short> siter(1);
    thrust::copy(siter, siter + 4, hvec.begin());
    ASSERT_TRUE(same(hvec, hv<short>({1, 2, 3, 4})));
  }

  g_test = "CopyZipIterator";
  {
    thrust::device_vector<int> v1(hv<int>({1, 2, 3})), v2(hv<int>({4, 5, 6})), v3(3, 0), v4(3, 0);
    thrust::copy(thrust::make_zip_iterator(thrust::make_tuple(v1.begin(), v2.begin())),
                 thrust::make_zip_iterator(thrust::make_tuple(v1.end(), v2.end())),
                 thrust::make_zip_iterator(thrust::make_tuple(v3.begin(), v4.begin())));
    ASSERT_TRUE(same(to_host(v3), to_host(v1)));
    ASSERT_TRUE(same(to_host(v4), to_host(v2)));
    thrust::host_vector<int> h1(hv<int>({1, 2, 3})), h2(hv<int>({4, 5, 6})), h3(3, 0), h4(3, 0);
    thrust::copy(thrust::make_zip_iterator(thrust::make_tuple(h1.begin(), h2.begin())),
                 thrust::make_zip_iterator(thrust::make_tuple(h1.end(), h2.end())),
                 thrust::make_zip_iterator(thrust::make_tuple(h3.begin(), h4.begin())));
    ASSERT_TRUE(same(h3, h1) && same(h4, h2));
  }

  g_test = "CopyConstantIteratorToZipIterator";
  {
    thrust::device_vector<int> v1(3, 0), v2(3, 0);
    thrust::copy(thrust::make_constant_iterator(thrust::tuple<int, int>(4, 7)),
                 thrust::make_constant_iterator(thrust::tuple<int, int>(4, 7)) + v1.size(),
                 thrust::make_zip_iterator(thrust::make_tuple(v1.begin(), v2.begin())));
    ASSERT_TRUE(same(to_host(v1), hv<int>({4, 4, 4})));
    ASSERT_TRUE(same(to_host(v2), hv<int>({7, 7, 7})));
  }
}

// ------------------------------------------------------------------ copy_if
template <typename T>
struct is_even {
  __host__ __device__ bool operator()(T x) { return (x & 1) == 0; }
};
template <typename T>
struct is_true {
  __host__ __device__ bool operator()(T x) { return x ? true : false; }
};
template <typename T>
struct mod_3 {
  __host__ __device__ unsigned int operator()(T x) { return x % 3; }
};

template <typename T, typename Pred>
static void copy_if_against_host(const thrust::host_vector<T>& h_data, Pred pred) {
  const size_t n = h_data.size();
  thrust::device_vector<T> d_data = h_data;
  thrust::host_vector<T> h_result(n);
  thrust::device_vector<T> d_result(n);
  auto h_end = thrust::copy_if(h_data.begin(), h_data.end(), h_result.begin(), pred);
  auto d_end = thrust::copy_if(d_data.begin(), d_data.end(), d_result.begin(), pred);
  h_result.resize(h_end - h_result.begin());
  d_result.resize(d_end - d_result.begin());
  ASSERT_TRUE(same(to_host(d_result), h_result));
  std::vector<T> expect;
  for (size_t i = 0; i < n; ++i)
    if (pred(h_data[i])) expect.push_back(h_data[i]);
  ASSERT_TRUE(same(h_result, expect));
}

template <typename T>
static void CopyIfForType(uint64_t seed) {
  for (size_t n : kSizes) {
    thrust::host_vector<T> random = random_integers<T>(n, seed + n);
    copy_if_against_host(random, is_true<T>());
    copy_if_against_host(random, is_even<T>());
    copy_if_against_host(random, mod_3<T>());  // a predicate that returns a number, not a bool
    thrust::host_vector<T> seq(n);
    thrust::sequence(seq.begin(), seq.end());
    thrust::device_vector<T> dseq(n);
    thrust::sequence(dseq.begin(), dseq.end());
    ASSERT_TRUE(same(to_host(dseq), seq));
    copy_if_against_host(seq, is_even<T>());
    copy_if_against_host(seq, mod_3<T>());
    // by a random stencil of the same type
    thrust::host_vector<T> h_stencil = random_integers<T>(n, seed + 77 + n);
    thrust::device_vector<T> d_stencil = h_stencil;
    thrust::host_vector<T> h_result(n);
    thrust::device_vector<T> d_result(n);
    auto h_end = thrust::copy_if(seq.begin(), seq.end(), h_stencil.begin(), h_result.begin(), is_even<T>());
    auto d_end = thrust::copy_if(dseq.begin(), dseq.end(), d_stencil.begin(), d_result.begin(), is_even<T>());
    h_result.resize(h_end - h_result.begin());
    d_result.resize(d_end - d_result.begin());
    ASSERT_TRUE(same(to_host(d_result), h_result));
  }
}

static void TestCopyIfPredicatesAndStencils() {
  g_test = "CopyIfIntegral / Sequence / Stencil";
  CopyIfForType<signed char>(1);
  CopyIfForType<unsigned char>(2);
  CopyIfForType<short>(3);
  CopyIfForType<unsigned short>(4);
  CopyIfForType<int>(5);
  CopyIfForType<unsigned int>(6);
  CopyIfForType<long long>(7);
  CopyIfForType<unsigned long long>(8);
  g_test = "CopyIfSimple";
  {
    thrust::device_vector<int> v(hv<int>({0, 1, 2, 3, 4})), dest(4);
    auto end = thrust::copy_if(v.begin(), v.end(), dest.begin(), is_true<int>());
    ASSERT_TRUE(end == dest.end());
    ASSERT_TRUE(same(to_host(dest), hv<int>({1, 2, 3, 4})));
    thrust::device_vector<int> s(hv<int>({1, 1, 0, 1, 0})), dest3(3);
    auto end3 = thrust::copy_if(v.begin(), v.end(), s.begin(), dest3.begin(), is_true<int>());
    ASSERT_TRUE(end3 == dest3.end());
    ASSERT_TRUE(same(to_host(dest3), hv<int>({0, 1, 3})));
  }
}

// Assignment copies the field only into an object whose constructor has run.
struct object_with_non_trivial_ctor {
  static constexpr int MAGIC = 923390;
  int field;
  int magic;
  __host__ __device__ object_with_non_trivial_ctor() : field(0), magic(MAGIC) {}
  __host__ __device__ object_with_non_trivial_ctor(int f) : field(f), magic(MAGIC) {}
  object_with_non_trivial_ctor(const object_with_non_trivial_ctor&) = default;
  __host__ __device__ object_with_non_trivial_ctor& operator=(const object_with_non_trivial_ctor& x) {
    if (magic == MAGIC) field = x.field;
    return *this;
  }
};
struct always_true {
  __host__ __device__ bool operator()(const object_with_non_trivial_ctor&) { return true; }
};

static void TestCopyIfNonTrivial() {
  g_test = "CopyIfNonTrivial";
  thrust::device_vector<object_with_non_trivial_ctor> a(10, object_with_non_trivial_ctor(99));
  thrust::device_vector<object_with_non_trivial_ctor> b(10);
  auto end = thrust::copy_if(a.begin(), a.end(), b.begin(), always_true());
  ASSERT_TRUE(end == b.end());
  for (int i = 0; i < 10; ++i) {
    object_with_non_trivial_ctor ha(a[i]);
    object_with_non_trivial_ctor hb(b[i]);
    ASSERT_TRUE(ha.field == 99 && hb.field == 99 && hb.magic == object_with_non_trivial_ctor::MAGIC);
  }
}

// ------------------------------------------------------------------ discard_iterator as an output
template <typename K>
static void DiscardOutputsByKey(uint64_t seed) {
  typedef unsigned int V;
  for (size_t n : kSizes) {
    thrust::host_vector<K> h_keys = random_bools<K>(n, seed + n);
    thrust::host_vector<V> h_vals = random_integers<V>(n, seed + 99 + n);
    thrust::device_vector<K> d_keys = h_keys;
    thrust::device_vector<V> d_vals = h_vals;
    thrust::host_vector<K> unique_keys = h_keys;
    unique_keys.erase(thrust::unique(unique_keys.begin(), unique_keys.end()), unique_keys.end());
    const size_t runs = unique_keys.size();
    size_t count = n ? 1 : 0;
    for (size_t i = 1; i < n; ++i) count += h_keys[i] != h_keys[i - 1];
    ASSERT_TRUE(runs == count);
    // the full results, for what is not discarded
    thrust::host_vector<K> full_keys(n);
    thrust::host_vector<V> full_sums(n), full_firsts(n);
    thrust::reduce_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), full_keys.begin(), full_sums.begin());
    thrust::unique_by_key_copy(h_keys.begin(), h_keys.end(), h_vals.begin(), full_keys.begin(), full_firsts.begin());
    full_keys.resize(runs); full_sums.resize(runs); full_firsts.resize(runs);
    ASSERT_TRUE(same(full_keys, unique_keys));

    g_test = "ReduceByKeyToDiscardIterator";
    {
      thrust::host_vector<V> h_out(n);
      thrust::device_vector<V> d_out(n);
      auto h_end = thrust::reduce_by_key(h_keys.begin(), h_keys.end(), h_vals.begin(), thrust::make_discard_iterator(), h_out.begin());
      auto d_end = thrust::reduce_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), thrust::make_discard_iterator(), d_out.begin());
      ASSERT_TRUE((size_t)(h_end.second - h_out.begin()) == runs);
      ASSERT_TRUE((size_t)(d_end.second - d_out.begin()) == runs);
      ASSERT_TRUE(h_end.first == thrust::make_discard_iterator(runs));
      ASSERT_TRUE(d_end.first == thrust::make_discard_iterator(runs));
      h_out.resize(runs); d_out.resize(runs);
      ASSERT_TRUE(same(h_out, full_sums));
      ASSERT_TRUE(same(to_host(d_out), full_sums));
      // the sums discarded, the keys kept
      thrust::device_vector<K> d_kout(n);
      auto d_end2 = thrust::reduce_by_key(d_keys.begin(), d_keys.end(), d_vals.begin(), d_kout.begin(), thrust::make_discard_iterator());
      ASSERT_TRUE((size_t)(d_end2.first - d_kout.begin()) == runs);
      ASSERT_TRUE(d_end2.second == thrust::make_discard_iterator(runs));
      d_kout.resize(runs);
      ASSERT_TRUE(same(to_host(d_kout), unique_keys));
    }
    g_test = "UniqueCopyToDiscardIterator";
    {
      thrust::discard_iterator<> reference(runs);
      thrust::discard_iterator<> h_result = thrust::unique_copy(h_keys.begin(), h_keys.end(), thrust::make_discard_iterator());
      thrust::discard_iterator<> d_result = thrust::unique_copy(d_keys.begin(), d_keys.end(), thrust::make_discard_iterator());
      ASSERT_TRUE(reference == h_result);
      ASSERT_TRUE(reference == d_result);
    }
    g_test = "UniqueCopyByKeyToDiscardIterator";
    {
      auto h1 = thrust::unique_by_key_copy(h_keys.begin(), h_keys.end(), h_vals.begin(), thrust::make_discard_iterator(), thrust::make_discard_iterator());
      auto d1 = thrust::unique_by_key_copy(d_keys.begin(), d_keys.end(), d_vals.begin(), thrust::make_discard_iterator(), thrust::make_discard_iterator());
      ASSERT_TRUE(h1.first == thrust::make_discard_iterator(runs) && h1.second == thrust::make_discard_iterator(runs));
      ASSERT_TRUE(d1.first == thrust::make_discard_iterator(runs) && d1.second == thrust::make_discard_iterator(runs));
      // values discarded
      thrust::host_vector<K> h_kout(n);
      thrust::device_vector<K> d_kout(n);
      auto h2 = thrust::unique_by_key_copy(h_keys.begin(), h_keys.end(), h_vals.begin(), h_kout.begin(), thrust::make_discard_iterator());
      auto d2 = thrust::unique_by_key_copy(d_keys.begin(), d_keys.end(), d_vals.begin(), d_kout.begin(), thrust::make_discard_iterator());
      ASSERT_TRUE(h2.first == h_kout.begin() + runs && h2.second == thrust::make_discard_iterator(runs));
      ASSERT_TRUE(d2.first == d_kout.begin() + runs && d2.second == thrust::make_discard_iterator(runs));
      h_kout.resize(runs); d_kout.resize(runs);
      ASSERT_TRUE(same(h_kout, unique_keys));
      ASSERT_TRUE(same(to_host(d_kout), unique_keys));
      // keys discarded
      thrust::host_vector<V> h_vout(n);
      thrust::device_vector<V> d_vout(n);
      auto h3 = thrust::unique_by_key_copy(h_keys.begin(), h_keys.end(), h_vals.begin(), thrust::make_discard_iterator(), h_vout.begin());
      auto d3 = thrust::unique_by_key_copy(d_keys.begin(), d_keys.end(), d_vals.begin(), thrust::make_discard_iterator(), d_vout.begin());
      ASSERT_TRUE(h3.first == thrust::make_discard_iterator(runs) && h3.second == h_vout.begin() + runs);
      ASSERT_TRUE(d3.first == thrust::make_discard_iterator(runs) && d3.second == d_vout.begin() + runs);
      h_vout.resize(runs); d_vout.resize(runs);
      ASSERT_TRUE(same(h_vout, full_firsts));
      ASSERT_TRUE(same(to_host(d_vout), full_firsts));
    }
  }
}

template <typename T>
static void PartitionCopyToDiscard(uint64_t seed) {
  for (size_t n : kSizes) {
    thrust::host_vector<T> h_data = random_integers<T>(n, seed + n);
    thrust::device_vector<T> d_data = h_data;
    thrust::host_vector<T> h_stencil = random_integers<T>(n, seed + 31 + n);
    thrust::device_vector<T> d_stencil = h_stencil;
    for (int by_stencil = 0; by_stencil < 2; ++by_stencil) {
      const thrust::host_vector<T>& tested = by_stencil ? h_stencil : h_data;
      std::vector<T> trues, falses;
      for (size_t i = 0; i < n; ++i) ((tested[i] & 1) == 0 ? trues : falses).push_back(h_data[i]);
      const std::ptrdiff_t n_true = (std::ptrdiff_t)trues.size(), n_false = (std::ptrdiff_t)falses.size();
      for (int stable = 0; stable < 2; ++stable) {
        g_test = by_stencil ? (stable ? "StablePartitionCopyStencilToDiscardIterator" : "PartitionCopyStencilToDiscardIterator")
                            : (stable ? "StablePartitionCopyToDiscardIterator" : "PartitionCopyToDiscardIterator");
        auto run = [&](auto first, auto last, auto sten, auto out_true, auto out_false) {
          if (by_stencil)
            return stable ? thrust::stable_partition_copy(first, last, sten, out_true, out_false, is_even<T>())
                          : thrust::partition_copy(first, last, sten, out_true, out_false, is_even<T>());
          return stable ? thrust::stable_partition_copy(first, last, out_true, out_false, is_even<T>())
                        : thrust::partition_copy(first, last, out_true, out_false, is_even<T>());
        };
        // both outputs discarded
        auto h1 = run(h_data.begin(), h_data.end(), h_stencil.begin(), thrust::make_discard_iterator(), thrust::make_discard_iterator());
        auto d1 = run(d_data.begin(), d_data.end(), d_stencil.begin(), thrust::make_discard_iterator(), thrust::make_discard_iterator());
        ASSERT_TRUE(h1.first == thrust::make_discard_iterator(n_true) && h1.second == thrust::make_discard_iterator(n_false));
        ASSERT_TRUE(d1.first == thrust::make_discard_iterator(n_true) && d1.second == thrust::make_discard_iterator(n_false));
        // the rejected ones discarded
        thrust::host_vector<T> h_trues(n_true);
        thrust::device_vector<T> d_trues(n_true);
        auto h2 = run(h_data.begin(), h_data.end(), h_stencil.begin(), h_trues.begin(), thrust::make_discard_iterator());
        auto d2 = run(d_data.begin(), d_data.end(), d_stencil.begin(), d_trues.begin(), thrust::make_discard_iterator());
        ASSERT_TRUE(h2.first == h_trues.begin() + n_true && h2.second == thrust::make_discard_iterator(n_false));
        ASSERT_TRUE(d2.first == d_trues.begin() + n_true && d2.second == thrust::make_discard_iterator(n_false));
        ASSERT_TRUE(same(h_trues, trues));
        ASSERT_TRUE(same(to_host(d_trues), trues));
        // the selected ones discarded
        thrust::host_vector<T> h_falses(n_false);
        thrust::device_vector<T> d_falses(n_false);
        auto h3 = run(h_data.begin(), h_data.end(), h_stencil.begin(), thrust::make_discard_iterator(), h_falses.begin());
        auto d3 = run(d_data.begin(), d_data.end(), d_stencil.begin(), thrust::make_discard_iterator(), d_falses.begin());
        ASSERT_TRUE(h3.first == thrust::make_discard_iterator(n_true) && h3.second == h_falses.begin() + n_false);
        ASSERT_TRUE(d3.first == thrust::make_discard_iterator(n_true) && d3.second == d_falses.begin() + n_false);
        ASSERT_TRUE(same(h_falses, falses));
        ASSERT_TRUE(same(to_host(d_falses), falses));
      }
    }
  }
}

template <typename T>
struct max_functor {
  __host__ __device__ T operator()(T a, T b) const { return a < b ? b : a; }
};

static void TestScansToDiscardIterator() {
  g_test = "ScanToDiscardIterator";
  for (size_t n : kSizes) {
    thrust::host_vector<int> h = random_integers<int>(n, 400 + n);
    thrust::device_vector<int> d = h;
    thrust::discard_iterator<> reference(n);
    ASSERT_TRUE(thrust::inclusive_scan(h.begin(), h.end(), thrust::make_discard_iterator()) == reference);
    ASSERT_TRUE(thrust::inclusive_scan(d.begin(), d.end(), thrust::make_discard_iterator()) == reference);
    ASSERT_TRUE(thrust::exclusive_scan(h.begin(), h.end(), thrust::make_discard_iterator(), 11) == reference);
    ASSERT_TRUE(thrust::exclusive_scan(d.begin(), d.end(), thrust::make_discard_iterator(), 11) == reference);
    // with an operator of the test's own (testing/scan.cu:264-296)
    ASSERT_TRUE(thrust::inclusive_scan(h.begin(), h.end(), thrust::make_discard_iterator(), max_functor<int>()) == reference);
    ASSERT_TRUE(thrust::inclusive_scan(d.begin(), d.end(), thrust::make_discard_iterator(), max_functor<int>()) == reference);
    ASSERT_TRUE(thrust::exclusive_scan(h.begin(), h.end(), thrust::make_discard_iterator(), 13, max_functor<int>()) == reference);
    ASSERT_TRUE(thrust::exclusive_scan(d.begin(), d.end(), thrust::make_discard_iterator(), 13, max_functor<int>()) == reference);
  }
}

static void TestDiscardOutputs() {
  DiscardOutputsByKey<int>(100);
  DiscardOutputsByKey<unsigned char>(200);
  DiscardOutputsByKey<long long>(300);
  PartitionCopyToDiscard<int>(500);
  PartitionCopyToDiscard<unsigned short>(600);
  PartitionCopyToDiscard<long long>(700);
  TestScansToDiscardIterator();
}

// ------------------------------------------------------------------ zip iterators in partition
struct is_ordered {
  template <typename Tuple>
  __host__ __device__ bool operator()(const Tuple& t) const { return thrust::get<0>(t) <= thrust::get<1>(t); }
};

template <typename Vector>
static void PartitionZip() {
  typedef typename Vector::value_type T;
  auto vec = [](std::initializer_list<T> l) { return Vector(thrust::host_vector<T>(std::vector<T>(l))); };
  {
    g_test = "PartitionZipIterator";
    Vector data1 = vec({1, 2, 1, 1, 2}), data2 = vec({2, 1, 2, 2, 1});
    auto begin = thrust::make_zip_iterator(thrust::make_tuple(data1.begin(), data2.begin()));
    auto end = thrust::make_zip_iterator(thrust::make_tuple(data1.end(), data2.end()));
    auto iter = thrust::partition(begin, end, is_ordered());
    ASSERT_TRUE(iter - begin == 3);
    ASSERT_TRUE(same(thrust::host_vector<T>(data1), hv<T>({1, 1, 1, 2, 2})));
    ASSERT_TRUE(same(thrust::host_vector<T>(data2), hv<T>({2, 2, 2, 1, 1})));
  }
  {
    g_test = "PartitionStencilZipIterator";
    Vector data = vec({1, 0, 1, 1, 0}), stencil1 = vec({1, 2, 1, 1, 2}), stencil2 = vec({2, 1, 2, 2, 1});
    auto stencil_begin = thrust::make_zip_iterator(thrust::make_tuple(stencil1.begin(), stencil2.begin()));
    auto iter = thrust::partition(data.begin(), data.end(), stencil_begin, is_ordered());
    ASSERT_TRUE(iter - data.begin() == 3);
    ASSERT_TRUE(same(thrust::host_vector<T>(data), hv<T>({1, 1, 1, 0, 0})));
  }
  {
    g_test = "StablePartitionZipIterator";
    Vector data1 = vec({1, 2, 1, 1, 2}), data2 = vec({2, 0, 3, 2, 1});
    auto begin = thrust::make_zip_iterator(thrust::make_tuple(data1.begin(), data2.begin()));
    auto end = thrust::make_zip_iterator(thrust::make_tuple(data1.end(), data2.end()));
    auto iter = thrust::stable_partition(begin, end, is_ordered());
    ASSERT_TRUE(iter - begin == 3);
    ASSERT_TRUE(same(thrust::host_vector<T>(data1), hv<T>({1, 1, 1, 2, 2})));
    ASSERT_TRUE(same(thrust::host_vector<T>(data2), hv<T>({2, 3, 2, 0, 1})));
  }
  {
    g_test = "StablePartitionStencilZipIterator";
    Vector data = vec({1, 0, 1, 1, 0}), stencil1 = vec({1, 2, 1, 1, 2}), stencil2 = vec({2, 0, 3, 2, 1});
    auto stencil_begin = thrust::make_zip_iterator(thrust::make_tuple(stencil1.begin(), stencil2.begin()));
    auto mid = thrust::stable_partition(data.begin(), data.end(), stencil_begin, is_ordered());
    ASSERT_TRUE(mid - data.begin() == 3);
    ASSERT_TRUE(same(thrust::host_vector<T>(data), hv<T>({1, 1, 1, 0, 0})));
  }
}

static void TestPartitionZipIterators() {
  PartitionZip<thrust::host_vector<int> >();
  PartitionZip<thrust::device_vector<int> >();
  PartitionZip<thrust::device_vector<short> >();
  PartitionZip<thrust::device_vector<long long> >();
  // and at sizes beyond one tile, against the host system
  g_test = "StablePartitionZipIterator, large";
  for (size_t n : {(size_t)5000, (size_t)(1u << 18) + 7}) {
    thrust::host_vector<int> h1 = random_integers<int>(n, 900 + n), h2 = random_integers<int>(n, 901 + n);
    thrust::device_vector<int> d1 = h1, d2 = h2;
    auto hb = thrust::make_zip_iterator(thrust::make_tuple(h1.begin(), h2.begin()));
    auto db = thrust::make_zip_iterator(thrust::make_tuple(d1.begin(), d2.begin()));
    auto hm = thrust::stable_partition(hb, hb + n, is_ordered());
    auto dm = thrust::stable_partition(db, db + n, is_ordered());
    ASSERT_TRUE(hm - hb == dm - db);
    ASSERT_TRUE(same(to_host(d1), h1));
    ASSERT_TRUE(same(to_host(d2), h2));
  }
}

// ------------------------------------------------------------------ operators that read a table through a pointer
template <typename T>
struct plus_mod3 {
  T* table;
  __host__ __device__ T operator()(T a, T b) { return table[(int)(a + b)]; }
};

template <typename Vector>
static void WithIndirection() {
  typedef typename Vector::value_type T;
  auto vec = [](std::initializer_list<T> l) { return Vector(thrust::host_vector<T>(std::vector<T>(l))); };
  Vector data = vec({0, 1, 2, 1, 2, 0, 1});
  Vector table = vec({0, 1, 2, 0, 1, 2});
  g_test = "ReduceWithIndirection";
  T result = thrust::reduce(data.begin(), data.end(), T(0), plus_mod3<T>{thrust::raw_pointer_cast(&table[0])});
  ASSERT_TRUE(result == T(1));
  g_test = "InclusiveScanWithIndirection";
  thrust::inclusive_scan(data.begin(), data.end(), data.begin(), plus_mod3<T>{thrust::raw_pointer_cast(&table[0])});
  ASSERT_TRUE(same(thrust::host_vector<T>(data), hv<T>({0, 1, 0, 1, 0, 0, 1})));
}

static void TestIndirection() {
  WithIndirection<thrust::host_vector<int> >();
  WithIndirection<thrust::device_vector<int> >();
  WithIndirection<thrust::device_vector<signed char> >();
  WithIndirection<thrust::device_vector<unsigned short> >();
  WithIndirection<thrust::device_vector<unsigned long long> >();
  // the same operator over many tiles: a sum modulo 3 whatever the grouping
  g_test = "ScanWithIndirection, large";
  const size_t n = (1u << 18) + 7;
  thrust::host_vector<int> h(n);
  for (size_t i = 0; i < n; ++i) h[i] = (int)(mix(i) % 3);
  thrust::device_vector<int> d = h, table(hv<int>({0, 1, 2, 0, 1, 2})), out(n);
  plus_mod3<int> op{thrust::raw_pointer_cast(table.data())};
  thrust::inclusive_scan(d.begin(), d.end(), out.begin(), op);
  thrust::host_vector<int> got = out;
  bool ok = true;
  int running = 0;
  for (size_t i = 0; i < n; ++i) {
    running = (running + h[i]) % 3;
    ok = ok && got[i] == running;
  }
  ASSERT_TRUE(ok);
  ASSERT_TRUE(thrust::reduce(d.begin(), d.end(), 0, op) == running);
}

// ------------------------------------------------------------------ element types with their own operator+
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
  __host__ __device__ bool operator==(const FixedVector& o) const {
    for (unsigned int i = 0; i < N; ++i)
      if (!(data[i] == o.data[i])) return false;
    return true;
  }
};

template <typename T, unsigned int N>
static void ScanWithLargeTypes() {
  typedef FixedVector<T, N> E;
  const size_t n = (1024 * 1024) / sizeof(E);
  thrust::host_vector<E> h_input(n), h_output(n);
  for (size_t i = 0; i < n; ++i) h_input[i] = E(static_cast<T>(i));
  thrust::device_vector<E> d_input = h_input, d_output(n);
  thrust::inclusive_scan(h_input.begin(), h_input.end(), h_output.begin());
  thrust::inclusive_scan(d_input.begin(), d_input.end(), d_output.begin());
  ASSERT_TRUE(same(to_host(d_output), h_output));
  // element i of the inclusive scan holds 0 + 1 + .. + i in every slot (modulo 2^32)
  bool closed_form = true;
  for (size_t i = 0; i < n; i += 97) closed_form = closed_form && h_output[i] == E(static_cast<T>((uint64_t)i * (i + 1) / 2));
  ASSERT_TRUE(closed_form);
  thrust::exclusive_scan(h_input.begin(), h_input.end(), h_output.begin(), E(0));
  thrust::exclusive_scan(d_input.begin(), d_input.end(), d_output.begin(), E(0));
  ASSERT_TRUE(same(to_host(d_output), h_output));
}

struct Int {
  int i{};
  __host__ __device__ explicit Int(int num) : i(num) {}
  __host__ __device__ Int() : i{} {}
  __host__ __device__ Int operator+(Int const& o) const { return Int{this->i + o.i}; }
};

static void TestScanElementTypes() {
  g_test = "ScanWithLargeTypes";
  ScanWithLargeTypes<int, 1>();
  ScanWithLargeTypes<int, 8>();
  ScanWithLargeTypes<int, 64>();
  g_test = "InclusiveScanWithUserDefinedType";
  thrust::device_vector<Int> vec(5, Int{1});
  thrust::inclusive_scan(thrust::device, vec.cbegin(), vec.cend(), vec.begin());
  ASSERT_TRUE(static_cast<Int>(vec.back()).i == 5);
}

int main() {
  TestSortBool();
  TestSortByKeyBool();
  TestCopyStandardContainers();
  TestCopyToDiscardAndZip();
  TestCopyIfPredicatesAndStencils();
  TestCopyIfNonTrivial();
  TestDiscardOutputs();
  TestPartitionZipIterators();
  TestIndirection();
  TestScanElementTypes();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
