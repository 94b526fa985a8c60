// Front-end test compiled with hipcc: fancy iterators as inputs of the device system's
// algorithms, user functors in transform / for_each / transform_reduce / count_if /
// copy_if, and sequence / gather / scatter.  Literal vectors are the reference's
// (testing/gather.cu:14-32, scatter.cu:10-32, sequence.cu:43-76, transform.cu:11-28 and
// :261-280, counting_iterator.cu, constant_iterator.cu); everything else compares the
// device system with the sequential host system on the same inputs.
#include <thrust/copy.h>
#include <thrust/count.h>
#include <thrust/device_vector.h>
#include <thrust/execution_policy.h>
#include <thrust/for_each.h>
#include <thrust/functional.h>
#include <thrust/gather.h>
#include <thrust/host_vector.h>
#include <thrust/inner_product.h>
#include <thrust/async/for_each.h>
#include <thrust/async/transform.h>
#include <thrust/future.h>
#include <thrust/iterator/constant_iterator.h>
#include <thrust/iterator/discard_iterator.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/permutation_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/sort.h>
#include <thrust/tuple.h>
#include <thrust/partition.h>
#include <thrust/remove.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/scatter.h>
#include <thrust/sequence.h>
#include <thrust/transform.h>
#include <thrust/transform_reduce.h>
#include <thrust/unique.h>

#include <hip/hip_runtime.h>

#include <cstdint>
#include <algorithm>
#include <cstdio>
#include <utility>
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
static thrust::host_vector<T> random_values(size_t n, uint64_t seed, uint64_t modulus) {
  thrust::host_vector<T> h(n);
  for (size_t i = 0; i < n; ++i) h[i] = (T)(mix(seed * 1000003ull + i) % modulus);
  return h;
}

static const size_t kSizes[] = {0, 1, 2, 63, 64, 65, 255, 256, 257, 1000, 4095, 4096, 4097, 65533, 65536, 65539,
                                (1u << 20) + 3};

struct times_three_plus_one {
  __host__ __device__ int operator()(int x) const { return 3 * x + 1; }
};
struct saxpy {
  float a;
  __host__ __device__ float operator()(float x, float y) const { return a * x + y; }
};
struct is_even {
  __host__ __device__ bool operator()(int x) const { return (x & 1) == 0; }
};
struct double_in_place {
  __host__ __device__ void operator()(int& x) const { x = 2 * x + 1; }
};
struct widen_square {
  __host__ __device__ long long operator()(int x) const { return (long long)x * x; }
};

// an element wider than a lane's share of a tile: one element per lane in the scans
struct Wide {
  double v[12];
  __host__ __device__ bool operator==(const Wide& o) const {
    for (int i = 0; i < 12; ++i)
      if (v[i] != o.v[i]) return false;
    return true;
  }
};
struct add_wide {
  __host__ __device__ Wide operator()(const Wide& a, const Wide& b) const {
    Wide r;
    for (int i = 0; i < 12; ++i) r.v[i] = a.v[i] + b.v[i];
    return r;
  }
};
// user operators for reduce and the scans
struct Affine {  // x -> a * x + b over unsigned wrap-around; composition is associative, not commutative
  unsigned a, b;
  __host__ __device__ bool operator==(const Affine& o) const { return a == o.a && b == o.b; }
};
struct compose {  // apply the left function first, then the right one
  __host__ __device__ Affine operator()(const Affine& f, const Affine& g) const { return Affine{f.a * g.a, f.b * g.a + g.b}; }
};
struct MinMax {
  int lo, hi;
  __host__ __device__ bool operator==(const MinMax& o) const { return lo == o.lo && hi == o.hi; }
};
struct to_minmax {
  __host__ __device__ MinMax operator()(int x) const { return MinMax{x, x}; }
};
struct merge_minmax {  // associative and commutative
  __host__ __device__ MinMax operator()(const MinMax& a, const MinMax& b) const {
    return MinMax{a.lo < b.lo ? a.lo : b.lo, a.hi > b.hi ? a.hi : b.hi};
  }
};
struct bit_xor_op {
  __host__ __device__ unsigned operator()(unsigned a, unsigned b) const { return a ^ b; }
};

static void TestUserOperators() {
  for (size_t n : kSizes) {
    g_test = "reduce with user operators";
    {
      const thrust::host_vector<int> h = random_values<int>(n, 21, 100001);
      const thrust::device_vector<int> d(h);
      const MinMax init = {1 << 30, -(1 << 30)};
      // the minimum / maximum example of the reference (examples/minmax.cu): one pass, a struct as the sum
      const MinMax want = thrust::transform_reduce(h.begin(), h.end(), to_minmax(), init, merge_minmax());
      const MinMax got = thrust::transform_reduce(d.begin(), d.end(), to_minmax(), init, merge_minmax());
      ASSERT_TRUE(got == want);
      const thrust::host_vector<unsigned> hu = random_values<unsigned>(n, 22, 1u << 31);
      const thrust::device_vector<unsigned> du(hu);
      ASSERT_TRUE(thrust::reduce(du.begin(), du.end(), 5u, bit_xor_op()) == thrust::reduce(hu.begin(), hu.end(), 5u, bit_xor_op()));
      ASSERT_TRUE(thrust::reduce(du.begin(), du.end(), 1u, thrust::multiplies<unsigned>()) ==
                  thrust::reduce(hu.begin(), hu.end(), 1u, thrust::multiplies<unsigned>()));
    }
    g_test = "scans with user operators";
    {
      thrust::host_vector<Affine> h(n);
      for (size_t i = 0; i < n; ++i) h[i] = Affine{(unsigned)(mix(i) | 1u), (unsigned)mix(i + 99)};
      Affine* dptr = nullptr;
      Affine* dout = nullptr;
      if (n) {
        dptr = thrust::raw_pointer_cast(thrust::device_malloc<Affine>(n));
        dout = thrust::raw_pointer_cast(thrust::device_malloc<Affine>(n));
        (void)hipMemcpy(dptr, h.data(), n * sizeof(Affine), hipMemcpyHostToDevice);
      }
      thrust::host_vector<Affine> want(n), got(n);
      thrust::inclusive_scan(h.begin(), h.end(), want.begin(), compose());
      thrust::inclusive_scan(thrust::device, dptr, dptr + n, dout, compose());
      if (n) (void)hipMemcpy(got.data(), dout, n * sizeof(Affine), hipMemcpyDeviceToHost);
      ASSERT_TRUE(same(got, want));
      const Affine init = {3u, 7u};
      thrust::exclusive_scan(h.begin(), h.end(), want.begin(), init, compose());
      thrust::exclusive_scan(thrust::device, dptr, dptr + n, dout, init, compose());
      if (n) (void)hipMemcpy(got.data(), dout, n * sizeof(Affine), hipMemcpyDeviceToHost);
      ASSERT_TRUE(same(got, want));
      // in place
      thrust::inclusive_scan(h.begin(), h.end(), want.begin(), compose());
      thrust::inclusive_scan(thrust::device, dptr, dptr + n, dptr, compose());
      if (n) (void)hipMemcpy(got.data(), dptr, n * sizeof(Affine), hipMemcpyDeviceToHost);
      ASSERT_TRUE(same(got, want));
      if (n) {
        thrust::device_free(thrust::device_pointer_cast(dptr));
        thrust::device_free(thrust::device_pointer_cast(dout));
      }
      // an operator of thrust/functional.h outside the library's set, on arithmetic elements
      const thrust::host_vector<unsigned> hu = random_values<unsigned>(n, 23, 1u << 31);
      const thrust::device_vector<unsigned> du(hu);
      thrust::host_vector<unsigned> hs(n);
      thrust::device_vector<unsigned> ds(n);
      thrust::inclusive_scan(hu.begin(), hu.end(), hs.begin(), thrust::multiplies<unsigned>());
      thrust::inclusive_scan(du.begin(), du.end(), ds.begin(), thrust::multiplies<unsigned>());
      ASSERT_TRUE(same(to_host(ds), hs));
      thrust::exclusive_scan(hu.begin(), hu.end(), hs.begin(), 9u, bit_xor_op());
      thrust::exclusive_scan(du.begin(), du.end(), ds.begin(), 9u, bit_xor_op());
      ASSERT_TRUE(same(to_host(ds), hs));
    }
  }
}

// Ranges of more than 32 MiB take the large tile shape of the single-pass scan (1024 threads x 12
// vectors): the same checks there, for an operator that does not commute on 8-byte elements and
// for one of thrust/functional.h on 4-byte elements.
static void TestUserOperatorScansOfLargeRanges() {
  g_test = "scans of large ranges with user operators";
  {
    const size_t n = ((size_t)1 << 23) + 12345;
    thrust::host_vector<Affine> h(n), want(n);
    for (size_t i = 0; i < n; ++i) h[i] = Affine{(unsigned)(mix(i) | 1u), (unsigned)mix(i + 99)};
    thrust::device_vector<Affine> d(h), out(n);
    thrust::inclusive_scan(h.begin(), h.end(), want.begin(), compose());
    thrust::inclusive_scan(d.begin(), d.end(), out.begin(), compose());
    ASSERT_TRUE(same(to_host(out), want));
    const Affine init = {5u, 11u};
    thrust::exclusive_scan(h.begin(), h.end(), want.begin(), init, compose());
    thrust::exclusive_scan(d.begin(), d.end(), d.begin(), init, compose());  // in place
    ASSERT_TRUE(same(to_host(d), want));
  }
  {
    const size_t n = ((size_t)1 << 23) + 7;
    const thrust::host_vector<unsigned> h = random_values<unsigned>(n, 41, 1u << 31);
    thrust::host_vector<unsigned> want(n);
    thrust::device_vector<unsigned> d(h), out(n);
    thrust::inclusive_scan(h.begin(), h.end(), want.begin(), thrust::multiplies<unsigned>());
    thrust::inclusive_scan(d.begin(), d.end(), out.begin(), thrust::multiplies<unsigned>());
    ASSERT_TRUE(same(to_host(out), want));
    thrust::exclusive_scan(h.begin(), h.end(), want.begin(), 3u, bit_xor_op());
    thrust::exclusive_scan(d.begin(), d.end(), out.begin(), 3u, bit_xor_op());
    ASSERT_TRUE(same(to_host(out), want));
  }
}

struct same_tens {  // the key predicate of testing/reduce_by_key.cu:60-112 and unique.cu:125-142
  __host__ __device__ bool operator()(int a, int b) const { return a / 10 == b / 10; }
};

static void TestWideElements() {
  g_test = "WideElements";
  for (size_t n : {(size_t)1, (size_t)255, (size_t)256, (size_t)257, (size_t)5000}) {
    thrust::host_vector<Wide> h(n);
    for (size_t i = 0; i < n; ++i)
      for (int k = 0; k < 12; ++k) h[i].v[k] = (double)((mix(i * 12 + k) % 1000));  // sums of integers: exact
    thrust::device_vector<Wide> d(h), dout(n);
    thrust::host_vector<Wide> hout(n);
    thrust::inclusive_scan(h.begin(), h.end(), hout.begin(), add_wide());
    thrust::inclusive_scan(d.begin(), d.end(), dout.begin(), add_wide());
    ASSERT_TRUE(same(to_host(dout), hout));
    Wide zero;
    for (int k = 0; k < 12; ++k) zero.v[k] = 1.0;
    thrust::exclusive_scan(h.begin(), h.end(), hout.begin(), zero, add_wide());
    thrust::exclusive_scan(d.begin(), d.end(), d.begin(), zero, add_wide());  // in place
    ASSERT_TRUE(same(to_host(d), hout));
  }
}

static void TestUserPredicatesByKey() {
  g_test = "by-key known answers with a user predicate";
  {
    // testing/unique.cu:105-142: [11,11,12,20,29,21,21,31,31,37] with "same tens" -> [11,20,31]
    thrust::device_vector<int> d(hv<int>({11, 11, 12, 20, 29, 21, 21, 31, 31, 37}));
    auto end = thrust::unique(d.begin(), d.end(), same_tens());
    ASSERT_TRUE(end - d.begin() == 3);
    d.resize(3);
    ASSERT_TRUE(same(to_host(d), hv<int>({11, 20, 31})));
    // testing/reduce_by_key.cu:60-112: keys [11,11,21,20,21,21,21,37,37], values 0..8, "same tens" -> [11,21,37] / [1,20,15]
    thrust::device_vector<int> k(hv<int>({11, 11, 21, 20, 21, 21, 21, 37, 37})), v(hv<int>({0, 1, 2, 3, 4, 5, 6, 7, 8}));
    thrust::device_vector<int> ko(9), vo(9);
    auto r = thrust::reduce_by_key(k.begin(), k.end(), v.begin(), ko.begin(), vo.begin(), same_tens());
    ASSERT_TRUE(r.first - ko.begin() == 3 && r.second - vo.begin() == 3);
    ko.resize(3); vo.resize(3);
    ASSERT_TRUE(same(to_host(ko), hv<int>({11, 21, 37})));
    ASSERT_TRUE(same(to_host(vo), hv<int>({1, 20, 15})));
    // testing/unique_by_key.cu:160-253 with the same predicate -> keys [11,21,37], values [0,2,7]
    thrust::device_vector<int> k2(k), v2(v);
    auto u = thrust::unique_by_key(k2.begin(), k2.end(), v2.begin(), same_tens());
    ASSERT_TRUE(u.first - k2.begin() == 3);
    k2.resize(3); v2.resize(3);
    ASSERT_TRUE(same(to_host(k2), hv<int>({11, 21, 37})));
    ASSERT_TRUE(same(to_host(v2), hv<int>({0, 2, 7})));
  }
  for (size_t n : kSizes) {
    g_test = "by-key differentials with user predicate and operator";
    thrust::host_vector<int> hk(n);
    for (size_t i = 0; i < n; ++i) hk[i] = (int)(i / 2 + mix(i / 5) % 7);
    const thrust::host_vector<unsigned> hvv = random_values<unsigned>(n, 31, 1u << 20);
    const thrust::device_vector<int> dk(hk);
    const thrust::device_vector<unsigned> dv(hvv);
    thrust::host_vector<int> hko(n);
    thrust::host_vector<unsigned> hvo(n);
    thrust::device_vector<int> dko(n);
    thrust::device_vector<unsigned> dvo(n);
    auto hr = thrust::reduce_by_key(hk.begin(), hk.end(), hvv.begin(), hko.begin(), hvo.begin(), same_tens(), bit_xor_op());
    auto dr = thrust::reduce_by_key(dk.begin(), dk.end(), dv.begin(), dko.begin(), dvo.begin(), same_tens(), bit_xor_op());
    ASSERT_TRUE(dr.first - dko.begin() == hr.first - hko.begin());
    size_t runs = hr.first - hko.begin();
    hko.resize(runs); hvo.resize(runs); dko.resize(runs); dvo.resize(runs);
    ASSERT_TRUE(same(to_host(dko), hko));
    ASSERT_TRUE(same(to_host(dvo), hvo));
    // equal_to with an operator outside the library's set
    hko.resize(n); hvo.resize(n); dko.resize(n); dvo.resize(n);
    hr = thrust::reduce_by_key(hk.begin(), hk.end(), hvv.begin(), hko.begin(), hvo.begin(), thrust::equal_to<int>(),
                               thrust::multiplies<unsigned>());
    dr = thrust::reduce_by_key(dk.begin(), dk.end(), dv.begin(), dko.begin(), dvo.begin(), thrust::equal_to<int>(),
                               thrust::multiplies<unsigned>());
    runs = hr.first - hko.begin();
    ASSERT_TRUE((size_t)(dr.first - dko.begin()) == runs);
    hko.resize(runs); hvo.resize(runs); dko.resize(runs); dvo.resize(runs);
    ASSERT_TRUE(same(to_host(dko), hko));
    ASSERT_TRUE(same(to_host(dvo), hvo));
    // scan_by_key with a user key predicate and operator (inclusive, exclusive with init, in place)
    {
      thrust::host_vector<unsigned> hs(n);
      thrust::device_vector<unsigned> ds(n);
      thrust::inclusive_scan_by_key(hk.begin(), hk.end(), hvv.begin(), hs.begin(), same_tens(), bit_xor_op());
      thrust::inclusive_scan_by_key(dk.begin(), dk.end(), dv.begin(), ds.begin(), same_tens(), bit_xor_op());
      ASSERT_TRUE(same(to_host(ds), hs));
      thrust::exclusive_scan_by_key(hk.begin(), hk.end(), hvv.begin(), hs.begin(), 7u, same_tens(), thrust::multiplies<unsigned>());
      thrust::exclusive_scan_by_key(dk.begin(), dk.end(), dv.begin(), ds.begin(), 7u, same_tens(), thrust::multiplies<unsigned>());
      ASSERT_TRUE(same(to_host(ds), hs));
      thrust::host_vector<unsigned> hin(hvv);
      thrust::device_vector<unsigned> din(dv);
      thrust::exclusive_scan_by_key(hk.begin(), hk.end(), hin.begin(), hin.begin(), 3u, thrust::equal_to<int>(), bit_xor_op());
      thrust::exclusive_scan_by_key(dk.begin(), dk.end(), din.begin(), din.begin(), 3u, thrust::equal_to<int>(), bit_xor_op());
      ASSERT_TRUE(same(to_host(din), hin));
      hin = hvv;
      din = dv;
      thrust::inclusive_scan_by_key(hk.begin(), hk.end(), hin.begin(), hin.begin(), same_tens(), bit_xor_op());
      thrust::inclusive_scan_by_key(dk.begin(), dk.end(), din.begin(), din.begin(), same_tens(), bit_xor_op());
      ASSERT_TRUE(same(to_host(din), hin));
    }
    // unique_copy and unique_by_key_copy
    hko.resize(n); dko.resize(n); hvo.resize(n); dvo.resize(n);
    auto he = thrust::unique_copy(hk.begin(), hk.end(), hko.begin(), same_tens());
    auto de = thrust::unique_copy(dk.begin(), dk.end(), dko.begin(), same_tens());
    ASSERT_TRUE(de - dko.begin() == he - hko.begin());
    hko.resize(he - hko.begin()); dko.resize(de - dko.begin());
    ASSERT_TRUE(same(to_host(dko), hko));
    hko.resize(n); dko.resize(n);
    auto hu = thrust::unique_by_key_copy(hk.begin(), hk.end(), hvv.begin(), hko.begin(), hvo.begin(), same_tens());
    auto du = thrust::unique_by_key_copy(dk.begin(), dk.end(), dv.begin(), dko.begin(), dvo.begin(), same_tens());
    runs = hu.first - hko.begin();
    ASSERT_TRUE((size_t)(du.first - dko.begin()) == runs);
    hko.resize(runs); hvo.resize(runs); dko.resize(runs); dvo.resize(runs);
    ASSERT_TRUE(same(to_host(dko), hko));
    ASSERT_TRUE(same(to_host(dvo), hvo));
  }
}

// reduce_by_key through the single-pass kernel instantiated for the caller's functors: operators
// without an identity that are not commutative (so any change of order or a stray operand
// shows), struct values, struct keys, narrow values, and runs from one element to several tiles.
struct span {  // the range of positions a run covers, and how many elements it has
  int first, last;
  __host__ __device__ bool operator==(const span& o) const { return first == o.first && last == o.last; }
};
struct join_spans {  // associative, not commutative, no identity
  __host__ __device__ span operator()(const span& a, const span& b) const { return span{a.first, b.last}; }
};
struct take_right {
  __host__ __device__ unsigned operator()(unsigned, unsigned b) const { return b; }
};
struct affine {  // x -> a x + b over the integers modulo 2^32; composition is associative, not commutative
  unsigned a, b;
  __host__ __device__ bool operator==(const affine& o) const { return a == o.a && b == o.b; }
};
struct compose_affine {
  __host__ __device__ affine operator()(const affine& f, const affine& g) const { return affine{g.a * f.a, g.a * f.b + g.b}; }
};
struct wide_key {
  int group;
  int noise;
  __host__ __device__ bool operator==(const wide_key& o) const { return group == o.group && noise == o.noise; }
};
struct same_group {
  __host__ __device__ bool operator()(const wide_key& a, const wide_key& b) const { return a.group == b.group; }
};
struct short_max {
  __host__ __device__ short operator()(short a, short b) const { return a < b ? b : a; }
};

template <typename K, typename V, typename Eq, typename Op>
static void CheckReduceByKey(const thrust::host_vector<K>& hk, const thrust::host_vector<V>& hval, Eq eq, Op op) {
  const size_t n = hk.size();
  const thrust::device_vector<K> dk(hk);
  const thrust::device_vector<V> dval(hval);
  thrust::host_vector<K> hko(n);
  thrust::host_vector<V> hvo(n);
  thrust::device_vector<K> dko(n);
  thrust::device_vector<V> dvo(n);
  auto hr = thrust::reduce_by_key(hk.begin(), hk.end(), hval.begin(), hko.begin(), hvo.begin(), eq, op);
  auto dr = thrust::reduce_by_key(dk.begin(), dk.end(), dval.begin(), dko.begin(), dvo.begin(), eq, op);
  const size_t runs = hr.first - hko.begin();
  ASSERT_TRUE((size_t)(dr.first - dko.begin()) == runs && (size_t)(dr.second - dvo.begin()) == runs);
  ASSERT_TRUE(same(thrust::host_vector<K>(dko.begin(), dko.begin() + runs), thrust::host_vector<K>(hko.begin(), hko.begin() + runs)));
  ASSERT_TRUE(same(thrust::host_vector<V>(dvo.begin(), dvo.begin() + runs), thrust::host_vector<V>(hvo.begin(), hvo.begin() + runs)));
  // the segmented scans over the same runs: inclusive, exclusive with an init, exclusive in place
  if (n == 0) return;
  thrust::inclusive_scan_by_key(hk.begin(), hk.end(), hval.begin(), hvo.begin(), eq, op);
  thrust::inclusive_scan_by_key(dk.begin(), dk.end(), dval.begin(), dvo.begin(), eq, op);
  ASSERT_TRUE(same(to_host(dvo), hvo));
  const V init = hval[n / 2];
  thrust::exclusive_scan_by_key(hk.begin(), hk.end(), hval.begin(), hvo.begin(), init, eq, op);
  thrust::exclusive_scan_by_key(dk.begin(), dk.end(), dval.begin(), dvo.begin(), init, eq, op);
  ASSERT_TRUE(same(to_host(dvo), hvo));
  thrust::device_vector<V> din(dval);
  thrust::exclusive_scan_by_key(dk.begin(), dk.end(), din.begin(), din.begin(), init, eq, op);
  ASSERT_TRUE(same(to_host(din), hvo));
}

static void TestReduceByKeyWithUserFunctors() {
  g_test = "reduce_by_key and scan_by_key with user functors in the single-pass kernels";
  for (size_t n : {(size_t)1, (size_t)2, (size_t)100, (size_t)14336, (size_t)14337, (size_t)100000, ((size_t)1 << 20) + 11}) {
    for (size_t mean_run : {(size_t)1, (size_t)3, (size_t)700, (size_t)50000, n + 1}) {
      thrust::host_vector<int> hk(n);
      thrust::host_vector<wide_key> hw(n);
      thrust::host_vector<span> hspan(n);
      thrust::host_vector<unsigned> hu(n);
      thrust::host_vector<affine> haff(n);
      thrust::host_vector<short> hsh(n);
      int group = 0;
      for (size_t i = 0; i < n; ++i) {
        if (i && mix(i * 7 + mean_run) % mean_run == 0) ++group;
        hk[i] = group;
        hw[i] = wide_key{group, (int)(mix(i) % 5)};
        hspan[i] = span{(int)i, (int)i};
        hu[i] = (unsigned)mix(i + 3);
        haff[i] = affine{(unsigned)(mix(i) | 1u), (unsigned)mix(i + 17)};
        hsh[i] = (short)(mix(i + 23) % 30000);
      }
      CheckReduceByKey(hk, hspan, thrust::equal_to<int>(), join_spans());
      CheckReduceByKey(hk, hu, thrust::equal_to<int>(), take_right());
      CheckReduceByKey(hw, haff, same_group(), compose_affine());
      CheckReduceByKey(hw, hu, same_group(), thrust::bit_xor<unsigned>());
      CheckReduceByKey(hk, hsh, thrust::equal_to<int>(), short_max());
    }
  }
}

struct add_first_two_into_third {  // the functor of examples/arbitrary_transformation.cu
  template <typename Tuple>
  __host__ __device__ void operator()(Tuple t) const { thrust::get<2>(t) = thrust::get<0>(t) + thrust::get<1>(t); }
};
struct swap_pair {
  __host__ __device__ thrust::tuple<float, int> operator()(const thrust::tuple<int, float>& t) const {
    return thrust::make_tuple(thrust::get<1>(t) * 2.0f, thrust::get<0>(t) + 1);
  }
};
struct tuple_sum {
  __host__ __device__ thrust::tuple<int, int> operator()(const thrust::tuple<int, int>& a, const thrust::tuple<int, int>& b) const {
    return thrust::make_tuple(thrust::get<0>(a) + thrust::get<0>(b), thrust::get<1>(a) + thrust::get<1>(b));
  }
};

static void TestZipIterator() {
  g_test = "ZipSimple";
  {
    // testing/zip_iterator.cu: dereference, arithmetic, assignment through the tuple of references
    thrust::device_vector<int> a(hv<int>({1, 2, 3, 4})), b(hv<int>({10, 20, 30, 40})), c(4, 0);
    auto z = thrust::make_zip_iterator(thrust::make_tuple(a.begin(), b.begin(), c.begin()));
    ASSERT_TRUE((z + 4) - z == 4);
    thrust::tuple<int, int, int> second = z[1];
    ASSERT_TRUE(thrust::get<0>(second) == 2 && thrust::get<1>(second) == 20 && thrust::get<2>(second) == 0);
    thrust::for_each(z, z + 4, add_first_two_into_third());
    ASSERT_TRUE(same(to_host(c), hv<int>({11, 22, 33, 44})));
    // sort_by_key with two value arrays zipped
    thrust::device_vector<int> keys(hv<int>({3, 1, 2, 1}));
    thrust::sort_by_key(keys.begin(), keys.end(), thrust::make_zip_iterator(thrust::make_tuple(a.begin(), b.begin())));
    ASSERT_TRUE(same(to_host(keys), hv<int>({1, 1, 2, 3})));
    ASSERT_TRUE(same(to_host(a), hv<int>({2, 4, 3, 1})));
    ASSERT_TRUE(same(to_host(b), hv<int>({20, 40, 30, 10})));
    // sorting a structure of arrays lexicographically
    thrust::device_vector<int> major(hv<int>({2, 1, 2, 1, 0})), minor(hv<int>({5, 9, 1, 3, 7}));
    auto zz = thrust::make_zip_iterator(thrust::make_tuple(major.begin(), minor.begin()));
    thrust::sort(zz, zz + 5);
    ASSERT_TRUE(same(to_host(major), hv<int>({0, 1, 1, 2, 2})));
    ASSERT_TRUE(same(to_host(minor), hv<int>({7, 3, 9, 1, 5})));
  }
  for (size_t n : kSizes) {
    g_test = "ZipDifferential";
    const thrust::host_vector<int> hi = random_values<int>(n, 41, 1000);
    thrust::host_vector<float> hf(n);
    for (size_t i = 0; i < n; ++i) hf[i] = (float)(mix(i + 5) % 4096) / 16.0f;
    const thrust::device_vector<int> di(hi);
    const thrust::device_vector<float> df(hf);
    // transform from a zip to a zip
    thrust::host_vector<float> hof(n);
    thrust::host_vector<int> hoi(n);
    thrust::device_vector<float> dof(n);
    thrust::device_vector<int> doi(n);
    thrust::transform(thrust::make_zip_iterator(thrust::make_tuple(hi.begin(), hf.begin())),
                      thrust::make_zip_iterator(thrust::make_tuple(hi.end(), hf.end())),
                      thrust::make_zip_iterator(thrust::make_tuple(hof.begin(), hoi.begin())), swap_pair());
    thrust::transform(thrust::make_zip_iterator(thrust::make_tuple(di.begin(), df.begin())),
                      thrust::make_zip_iterator(thrust::make_tuple(di.end(), df.end())),
                      thrust::make_zip_iterator(thrust::make_tuple(dof.begin(), doi.begin())), swap_pair());
    ASSERT_TRUE(same(to_host(dof), hof));
    ASSERT_TRUE(same(to_host(doi), hoi));
    // reduce of zipped ranges with a user operator: two sums in one pass
    const thrust::tuple<int, int> zero = thrust::make_tuple(0, 0);
    auto hz = thrust::make_zip_iterator(thrust::make_tuple(hi.begin(), hoi.begin()));
    auto dz = thrust::make_zip_iterator(thrust::make_tuple(di.begin(), doi.begin()));
    ASSERT_TRUE(thrust::reduce(dz, dz + n, zero, tuple_sum()) == thrust::reduce(hz, hz + n, zero, tuple_sum()));
    // stable sort of a structure of arrays by a user comparator on the tuple, against the host system
    thrust::host_vector<int> hk(hi), hv2(n);
    for (size_t i = 0; i < n; ++i) hv2[i] = (int)i;
    thrust::device_vector<int> dk(hk), dv2(hv2);
    auto hzz = thrust::make_zip_iterator(thrust::make_tuple(hk.begin(), hv2.begin()));
    auto dzz = thrust::make_zip_iterator(thrust::make_tuple(dk.begin(), dv2.begin()));
    thrust::sort(dzz, dzz + n);
    std::vector<std::pair<int, int> > ref(n);
    for (size_t i = 0; i < n; ++i) ref[i] = std::make_pair(hi[i], (int)i);
    std::sort(ref.begin(), ref.end());
    bool ok = true;
    const thrust::host_vector<int> gk = to_host(dk), gv = to_host(dv2);
    for (size_t i = 0; i < n; ++i) ok = ok && gk[i] == ref[i].first && gv[i] == ref[i].second;
    ASSERT_TRUE(ok);
    (void)hzz;
  }
}

// testing/reduce.cu:213-231: ranges of 2^30 .. 2^33 elements that exist only as an iterator
static void TestReduceWithBigIndexes() {
  g_test = "ReduceWithBigIndexes";
  for (int magnitude = 30; magnitude <= 33; ++magnitude) {
    thrust::constant_iterator<long long> begin(1);
    thrust::constant_iterator<long long> end = begin + (1ll << magnitude);
    ASSERT_TRUE(end - begin == (1ll << magnitude));
    const long long result = thrust::reduce(thrust::device, begin, end);
    ASSERT_TRUE(result == (1ll << magnitude));
  }
  // the same range counted: sum of 0 .. n-1
  const long long n = (1ll << 31) + 12345;
  thrust::counting_iterator<long long> first(0);
  const long long sum = thrust::reduce(thrust::device, first, first + n, 0ll);
  ASSERT_TRUE(sum == (long long)((unsigned long long)n * (unsigned long long)(n - 1) / 2));
}

// testing/scan.cu:563-663 and testing/copy.cu:713-781: ranges of 2^30 .. 2^33 elements that exist
// only as an iterator, written through an iterator of the test's own that remembers whether
// the one expected value came by.  Nothing is stored: only the 64-bit indexing is on trial.
struct only_set_when_expected_it {
  long long expected;
  bool* flag;
  __host__ __device__ only_set_when_expected_it operator++() const { return *this; }
  __host__ __device__ only_set_when_expected_it operator*() const { return *this; }
  template <typename Difference>
  __host__ __device__ only_set_when_expected_it operator+(Difference) const { return *this; }
  template <typename Difference>
  __host__ __device__ only_set_when_expected_it operator+=(Difference) const { return *this; }
  template <typename Index>
  __host__ __device__ only_set_when_expected_it operator[](Index) const { return *this; }
  __device__ void operator=(long long value) const {
    if (value == expected) *flag = true;
  }
};
namespace thrust {
template <>
struct iterator_traits<only_set_when_expected_it> {
  typedef long long value_type;
  typedef only_set_when_expected_it reference;
};
}  // namespace thrust

static void TestScanAndCopyWithBigIndexes() {
  g_test = "ScanAndCopyWithBigIndexes";
  thrust::device_vector<bool> flag(1);
  for (int magnitude = 30; magnitude <= 33; ++magnitude) {
    const long long n = 1ll << magnitude;
    thrust::constant_iterator<long long> ones(1);
    flag[0] = false;
    only_set_when_expected_it last_of_inclusive = {n, thrust::raw_pointer_cast(flag.data())};
    thrust::inclusive_scan(thrust::device, ones, ones + n, last_of_inclusive);
    ASSERT_TRUE((bool)flag[0]);
    flag[0] = false;
    only_set_when_expected_it last_of_exclusive = {n - 1, thrust::raw_pointer_cast(flag.data())};
    thrust::exclusive_scan(thrust::device, ones, ones + n, last_of_exclusive, 0ll);
    ASSERT_TRUE((bool)flag[0]);
    flag[0] = false;
    thrust::counting_iterator<long long> index(0);
    only_set_when_expected_it last_index = {n - 1, thrust::raw_pointer_cast(flag.data())};
    thrust::copy(thrust::device, index, index + n, last_index);
    ASSERT_TRUE((bool)flag[0]);
  }
  // a value that never comes by leaves the flag alone
  flag[0] = false;
  thrust::constant_iterator<long long> ones(1);
  only_set_when_expected_it never = {-5, thrust::raw_pointer_cast(flag.data())};
  thrust::inclusive_scan(thrust::device, ones, ones + (1ll << 20), never);
  ASSERT_TRUE(!(bool)flag[0]);
}

// thrust::discard_iterator as the output nobody wants, and an operator of another type than
// the elements: inclusive_scan of floats with plus<int> keeps the first element as it is and
// adds the others as integers (testing/scan.cu:257-262).
static void TestDiscardAndForeignOperator() {
  g_test = "DiscardIterator";
  {
    thrust::device_vector<int> d(hv<int>({1, 3, -2, 4, -5}));
    thrust::discard_iterator<> sink;
    auto end = thrust::inclusive_scan(thrust::device, d.begin(), d.end(), sink);
    ASSERT_TRUE(end - sink == 5);
    auto end2 = thrust::copy(thrust::device, thrust::counting_iterator<int>(0), thrust::counting_iterator<int>(1000), sink);
    ASSERT_TRUE(end2 - sink == 1000);
  }
  g_test = "ScanMixedTypesForeignOperator";
  {
    thrust::device_vector<float> in(hv<float>({1.5f, 2.5f, 3.5f, 4.5f})), out(4);
    thrust::inclusive_scan(in.begin(), in.end(), out.begin(), thrust::plus<int>());
    ASSERT_TRUE(same(to_host(out), hv<float>({1.5f, 3.0f, 6.0f, 10.0f})));
    thrust::host_vector<float> hin = in, hout(4);
    thrust::inclusive_scan(hin.begin(), hin.end(), hout.begin(), thrust::plus<int>());
    ASSERT_TRUE(same(hout, hv<float>({1.5f, 3.0f, 6.0f, 10.0f})));
  }
}

// thrust::async::for_each / transform with functors of the test's own, and when_all
// (testing/async_for_each.cu:20-60, testing/async_transform.cu:30-90: the asynchronous result
// equals the synchronous algorithm's; the event is waited for before the data is read).
struct add_seven { __host__ __device__ void operator()(int& x) const { x += 7; } };
struct times_three { __host__ __device__ long long operator()(int x) const { return 3ll * x; } };
static void TestAsyncForEachTransformWhenAll() {
  g_test = "AsyncForEachTransformWhenAll";
  for (size_t n : {(size_t)0, (size_t)1, (size_t)1000, ((size_t)1 << 20) + 3}) {
    thrust::host_vector<int> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = (int)(i * 2654435761u >> 8);
    thrust::device_vector<int> a = h, b = h;
    thrust::device_vector<long long> out(n);
    thrust::device_event e1 = thrust::async::for_each(a.begin(), a.end(), add_seven());
    thrust::device_event e2 = thrust::async::transform(thrust::device, b.begin(), b.end(), out.begin(), times_three());
    thrust::device_event both = thrust::when_all(e1, e2);
    both.wait();
    ASSERT_TRUE(both.ready());
    ASSERT_TRUE(e1.ready());
    e2.wait();
    ASSERT_TRUE(e2.ready());
    thrust::host_vector<int> ha = a;
    thrust::host_vector<long long> ho = out;
    bool ok = true;
    for (size_t i = 0; i < n; ++i) ok = ok && ha[i] == h[i] + 7 && ho[i] == 3ll * h[i];
    ASSERT_TRUE(ok);
    // chained: the transform starts after the for_each it depends on, on the same stream
    thrust::device_event e3 = thrust::async::for_each(a.begin(), a.end(), add_seven());
    void* s3 = e3.stream().native_handle();
    thrust::device_event e4 = thrust::async::transform(thrust::device.after(e3), a.begin(), a.end(), out.begin(), times_three());
    ASSERT_TRUE(e4.stream().native_handle() == s3);
    e4.wait();
    ho = out;
    ok = true;
    for (size_t i = 0; i < n; ++i) ok = ok && ho[i] == 3ll * (h[i] + 14);
    ASSERT_TRUE(ok);
  }
  thrust::device_event none = thrust::when_all();
  ASSERT_TRUE(none.ready());
  none.wait();
}

static void TestKnownAnswers() {
  g_test = "GatherSimple";
  {
    thrust::device_vector<int> map(hv<int>({6, 2, 1, 7, 2})), src(hv<int>({0, 1, 2, 3, 4, 5, 6, 7})), dst(5, 0);
    auto end = thrust::gather(map.begin(), map.end(), src.begin(), dst.begin());
    ASSERT_TRUE(end - dst.begin() == 5);
    ASSERT_TRUE(same(to_host(dst), hv<int>({6, 2, 1, 7, 2})));
  }
  g_test = "ScatterSimple";
  {
    thrust::device_vector<int> map(hv<int>({6, 3, 1, 7, 2})), src(hv<int>({0, 1, 2, 3, 4})), dst(8, 0);
    thrust::scatter(src.begin(), src.end(), map.begin(), dst.begin());
    ASSERT_TRUE(same(to_host(dst), hv<int>({0, 2, 4, 1, 0, 0, 0, 3})));
  }
  g_test = "SequenceSimple";
  {
    thrust::device_vector<int> v(5);
    thrust::sequence(v.begin(), v.end());
    ASSERT_TRUE(same(to_host(v), hv<int>({0, 1, 2, 3, 4})));
    thrust::sequence(v.begin(), v.end(), 10);
    ASSERT_TRUE(same(to_host(v), hv<int>({10, 11, 12, 13, 14})));
    thrust::sequence(v.begin(), v.end(), 10, 2);
    ASSERT_TRUE(same(to_host(v), hv<int>({10, 12, 14, 16, 18})));
  }
  g_test = "TransformSimple";
  {
    thrust::device_vector<int> in(hv<int>({1, -2, 3})), in2(hv<int>({-4, 5, 6})), out(3);
    auto it = thrust::transform(in.begin(), in.end(), out.begin(), thrust::negate<int>());
    ASSERT_TRUE(it - out.begin() == 3);
    ASSERT_TRUE(same(to_host(out), hv<int>({-1, 2, -3})));
    it = thrust::transform(in.begin(), in.end(), in2.begin(), out.begin(), thrust::minus<int>());
    ASSERT_TRUE(it - out.begin() == 3);
    ASSERT_TRUE(same(to_host(out), hv<int>({5, -7, -3})));
  }
  g_test = "CountingAndConstant";
  {
    thrust::counting_iterator<int> first(0);
    ASSERT_TRUE(*first == 0 && first[5] == 5 && (first + 3) - first == 3);
    ASSERT_TRUE(thrust::reduce(first, first + 100) == 4950);
    ASSERT_TRUE(thrust::reduce(thrust::device, first + 1, first + 4) == 6);  // testing/counting_iterator.cu sums 1 + 2 + 3
    thrust::constant_iterator<int> seven(7);
    ASSERT_TRUE(*seven == 7 && seven[12] == 7 && (seven + 9) - seven == 9);
    ASSERT_TRUE(thrust::reduce(seven, seven + 1000) == 7000);
    thrust::device_vector<int> out(4);
    thrust::copy(first + 3, first + 7, out.begin());
    ASSERT_TRUE(same(to_host(out), hv<int>({3, 4, 5, 6})));
    thrust::exclusive_scan(seven, seven + 4, out.begin());
    ASSERT_TRUE(same(to_host(out), hv<int>({0, 7, 14, 21})));
  }
}

static void Differential() {
  for (size_t n : kSizes) {
    const thrust::host_vector<int> h = random_values<int>(n, 3, 2001);
    const thrust::device_vector<int> d(h);

    g_test = "transform_iterator inputs";
    {
      auto hf = thrust::make_transform_iterator(h.begin(), times_three_plus_one());
      auto df = thrust::make_transform_iterator(d.begin(), times_three_plus_one());
      ASSERT_TRUE(thrust::reduce(df, df + n, 5) == thrust::reduce(hf, hf + n, 5));
      ASSERT_TRUE(thrust::reduce(df, df + n, -1000000, thrust::maximum<int>()) ==
                  thrust::reduce(hf, hf + n, -1000000, thrust::maximum<int>()));
      thrust::host_vector<int> hs(n);
      thrust::device_vector<int> ds(n);
      thrust::inclusive_scan(hf, hf + n, hs.begin());
      thrust::inclusive_scan(df, df + n, ds.begin());
      ASSERT_TRUE(same(to_host(ds), hs));
      thrust::exclusive_scan(hf, hf + n, hs.begin(), 11);
      thrust::exclusive_scan(df, df + n, ds.begin(), 11);
      ASSERT_TRUE(same(to_host(ds), hs));
    }
    g_test = "user functors";
    {
      ASSERT_TRUE(thrust::transform_reduce(d.begin(), d.end(), widen_square(), (long long)3, thrust::plus<long long>()) ==
                  thrust::transform_reduce(h.begin(), h.end(), widen_square(), (long long)3, thrust::plus<long long>()));
      ASSERT_TRUE(thrust::count_if(d.begin(), d.end(), is_even()) == thrust::count_if(h.begin(), h.end(), is_even()));
      thrust::host_vector<int> ho(n);
      thrust::device_vector<int> dout(n);
      auto he = thrust::copy_if(h.begin(), h.end(), ho.begin(), is_even());
      auto de = thrust::copy_if(d.begin(), d.end(), dout.begin(), is_even());
      ASSERT_TRUE(de - dout.begin() == he - ho.begin());
      ho.resize(he - ho.begin());
      dout.resize(de - dout.begin());
      ASSERT_TRUE(same(to_host(dout), ho));
      // stencil form: keep h[i] where the stencil is even
      const thrust::host_vector<int> hst = random_values<int>(n, 9, 10);
      const thrust::device_vector<int> dst(hst);
      ho.resize(n);
      dout.resize(n);
      he = thrust::copy_if(h.begin(), h.end(), hst.begin(), ho.begin(), is_even());
      de = thrust::copy_if(d.begin(), d.end(), dst.begin(), dout.begin(), is_even());
      ASSERT_TRUE(de - dout.begin() == he - ho.begin());
      ho.resize(he - ho.begin());
      dout.resize(de - dout.begin());
      ASSERT_TRUE(same(to_host(dout), ho));
    }
    g_test = "partition / remove_if with a user predicate";
    {
      thrust::host_vector<int> hp(h);
      thrust::device_vector<int> dp(d);
      auto hmid = thrust::stable_partition(hp.begin(), hp.end(), is_even());
      auto dmid = thrust::stable_partition(dp.begin(), dp.end(), is_even());
      ASSERT_TRUE(dmid - dp.begin() == hmid - hp.begin());
      ASSERT_TRUE(same(to_host(dp), hp));
      thrust::host_vector<int> ht(n), hf(n);
      thrust::device_vector<int> dt(n), df(n);
      auto hr = thrust::partition_copy(h.begin(), h.end(), ht.begin(), hf.begin(), is_even());
      auto dr = thrust::partition_copy(d.begin(), d.end(), dt.begin(), df.begin(), is_even());
      ASSERT_TRUE(dr.first - dt.begin() == hr.first - ht.begin() && dr.second - df.begin() == hr.second - hf.begin());
      ht.resize(hr.first - ht.begin()); hf.resize(hr.second - hf.begin());
      dt.resize(dr.first - dt.begin()); df.resize(dr.second - df.begin());
      ASSERT_TRUE(same(to_host(dt), ht));
      ASSERT_TRUE(same(to_host(df), hf));
      hp = h;
      dp = d;
      auto hend = thrust::remove_if(hp.begin(), hp.end(), is_even());
      auto dend = thrust::remove_if(dp.begin(), dp.end(), is_even());
      ASSERT_TRUE(dend - dp.begin() == hend - hp.begin());
      hp.resize(hend - hp.begin());
      dp.resize(dend - dp.begin());
      ASSERT_TRUE(same(to_host(dp), hp));
    }
    g_test = "transform / for_each / sequence";
    {
      thrust::host_vector<float> hx(n), hy(n), hz(n);
      for (size_t i = 0; i < n; ++i) { hx[i] = (float)(mix(i) % 1000) / 8.0f; hy[i] = (float)(mix(i + n) % 1000) / 4.0f; }
      thrust::device_vector<float> dx(hx), dy(hy), dz(n);
      thrust::transform(hx.begin(), hx.end(), hy.begin(), hz.begin(), saxpy{2.5f});
      thrust::transform(dx.begin(), dx.end(), dy.begin(), dz.begin(), saxpy{2.5f});
      ASSERT_TRUE(same(to_host(dz), hz));
      thrust::host_vector<int> h2(h);
      thrust::device_vector<int> d2(d);
      thrust::for_each(h2.begin(), h2.end(), double_in_place());
      thrust::for_each(d2.begin(), d2.end(), double_in_place());
      ASSERT_TRUE(same(to_host(d2), h2));
      thrust::transform(h.begin(), h.end(), h2.begin(), times_three_plus_one());
      thrust::transform(d.begin(), d.end(), d2.begin(), times_three_plus_one());
      ASSERT_TRUE(same(to_host(d2), h2));
      thrust::host_vector<long long> hq(n);
      thrust::device_vector<long long> dq(n);
      thrust::sequence(hq.begin(), hq.end(), (long long)-5, (long long)3);
      thrust::sequence(dq.begin(), dq.end(), (long long)-5, (long long)3);
      ASSERT_TRUE(same(to_host(dq), hq));
    }
    g_test = "gather / scatter / permutation";
    if (n) {
      // a permutation of 0..n-1: i -> (a*i + b) mod n with gcd(a, n) = 1
      size_t a = 7;
      while (a > 1 && (n % a == 0 || std::__gcd(a, n) != 1)) ++a;
      thrust::host_vector<unsigned> hmap(n);
      for (size_t i = 0; i < n; ++i) hmap[i] = (unsigned)((a * i + 3) % n);
      thrust::device_vector<unsigned> dmap(hmap);
      thrust::host_vector<int> hg(n), hsc(n, -1);
      thrust::device_vector<int> dg(n), dsc(n, -1);
      thrust::gather(hmap.begin(), hmap.end(), h.begin(), hg.begin());
      thrust::gather(dmap.begin(), dmap.end(), d.begin(), dg.begin());
      ASSERT_TRUE(same(to_host(dg), hg));
      thrust::scatter(h.begin(), h.end(), hmap.begin(), hsc.begin());
      thrust::scatter(d.begin(), d.end(), dmap.begin(), dsc.begin());
      ASSERT_TRUE(same(to_host(dsc), hsc));
      auto hp = thrust::make_permutation_iterator(h.begin(), hmap.begin());
      auto dp = thrust::make_permutation_iterator(d.begin(), dmap.begin());
      ASSERT_TRUE(thrust::reduce(dp, dp + n / 2, 1) == thrust::reduce(hp, hp + n / 2, 1));
    }
    g_test = "reduce_by_key with a constant iterator";
    {
      thrust::host_vector<int> hk(n);
      for (size_t i = 0; i < n; ++i) hk[i] = (int)(i / 3 + (mix(i / 3) % 2));
      thrust::device_vector<int> dk(hk), dko(n), dvo(n);
      thrust::host_vector<int> hko(n), hvo(n);
      auto hr = thrust::reduce_by_key(hk.begin(), hk.end(), thrust::constant_iterator<int>(1), hko.begin(), hvo.begin());
      auto dr = thrust::reduce_by_key(dk.begin(), dk.end(), thrust::constant_iterator<int>(1), dko.begin(), dvo.begin());
      ASSERT_TRUE(dr.first - dko.begin() == hr.first - hko.begin());
      const size_t runs = hr.first - hko.begin();
      hko.resize(runs); hvo.resize(runs); dko.resize(runs); dvo.resize(runs);
      ASSERT_TRUE(same(to_host(dko), hko));
      ASSERT_TRUE(same(to_host(dvo), hvo));
    }
    g_test = "inner_product with a counting iterator";
    {
      thrust::counting_iterator<int> c(1);
      long long want = 0;
      for (size_t i = 0; i < n; ++i) want += (long long)h[i] * (long long)(1 + (int)i);
      ASSERT_TRUE((long long)thrust::inner_product(d.begin(), d.end(), c, 0) == (long long)(int)want);
    }
  }
}

// Predicates, stencils and element structs of several widths through the selection kernel that is
// instantiated for them: every form against the host system on the same input, at sizes of
// several tiles, with most, half, few and none of the elements selected (the in-place partition
// sweeps from either end depending on that).
struct point {
  int x;
  float w;
  __host__ __device__ bool operator==(const point& o) const { return x == o.x && w == o.w; }
};
struct quad {  // a 16-byte stencil element
  int a, b, c, d;
};
struct below {
  int limit;
  __host__ __device__ bool operator()(int v) const { return v < limit; }
};
struct point_below {
  int limit;
  __host__ __device__ bool operator()(const point& p) const { return p.x < limit; }
};
struct quad_sum_below {
  int limit;
  __host__ __device__ bool operator()(const quad& q) const { return q.a + q.b + q.c + q.d < limit; }
};
struct byte_is_odd {
  __host__ __device__ bool operator()(unsigned char b) const { return (b & 1) != 0; }
};
struct double_below {
  double limit;
  __host__ __device__ bool operator()(double v) const { return v < limit; }
};
struct same_point_x {
  __host__ __device__ bool operator()(const point& a, const point& b) const { return a.x / 4 == b.x / 4; }
};

template <typename T, typename S, typename Pred>
static void CheckSelectionForms(const thrust::host_vector<T>& h, const thrust::host_vector<S>& hs, Pred pred) {
  const size_t n = h.size();
  const thrust::device_vector<T> d(h);
  const thrust::device_vector<S> ds(hs);
  thrust::host_vector<T> ho(n), hf(n);
  thrust::device_vector<T> dout(n), dfalse(n);
  {  // copy_if / remove_copy_if by stencil
    auto he = thrust::copy_if(h.begin(), h.end(), hs.begin(), ho.begin(), pred);
    auto de = thrust::copy_if(d.begin(), d.end(), ds.begin(), dout.begin(), pred);
    ASSERT_TRUE(de - dout.begin() == he - ho.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(dout.begin(), de), thrust::host_vector<T>(ho.begin(), he)));
    he = thrust::remove_copy_if(h.begin(), h.end(), hs.begin(), ho.begin(), pred);
    de = thrust::remove_copy_if(d.begin(), d.end(), ds.begin(), dout.begin(), pred);
    ASSERT_TRUE(de - dout.begin() == he - ho.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(dout.begin(), de), thrust::host_vector<T>(ho.begin(), he)));
  }
  {  // partition_copy by stencil
    auto hr = thrust::partition_copy(h.begin(), h.end(), hs.begin(), ho.begin(), hf.begin(), pred);
    auto dr = thrust::partition_copy(d.begin(), d.end(), ds.begin(), dout.begin(), dfalse.begin(), pred);
    ASSERT_TRUE(dr.first - dout.begin() == hr.first - ho.begin() && dr.second - dfalse.begin() == hr.second - hf.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(dout.begin(), dr.first), thrust::host_vector<T>(ho.begin(), hr.first)));
    ASSERT_TRUE(same(thrust::host_vector<T>(dfalse.begin(), dr.second), thrust::host_vector<T>(hf.begin(), hr.second)));
  }
  {  // stable_partition and remove_if in place, by stencil
    thrust::host_vector<T> hp(h);
    thrust::device_vector<T> dp(d);
    auto hm = thrust::stable_partition(hp.begin(), hp.end(), hs.begin(), pred);
    auto dm = thrust::stable_partition(dp.begin(), dp.end(), ds.begin(), pred);
    ASSERT_TRUE(dm - dp.begin() == hm - hp.begin());
    ASSERT_TRUE(same(to_host(dp), hp));
    hp = h;
    dp = d;
    auto hend = thrust::remove_if(hp.begin(), hp.end(), hs.begin(), pred);
    auto dend = thrust::remove_if(dp.begin(), dp.end(), ds.begin(), pred);
    ASSERT_TRUE(dend - dp.begin() == hend - hp.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(dp.begin(), dend), thrust::host_vector<T>(hp.begin(), hend)));
  }
}
template <typename T, typename Pred>
static void CheckSelectionOnTheElements(const thrust::host_vector<T>& h, Pred pred) {
  const size_t n = h.size();
  const thrust::device_vector<T> d(h);
  thrust::host_vector<T> ho(n), hf(n);
  thrust::device_vector<T> dout(n), dfalse(n);
  auto he = thrust::copy_if(h.begin(), h.end(), ho.begin(), pred);
  auto de = thrust::copy_if(d.begin(), d.end(), dout.begin(), pred);
  ASSERT_TRUE(de - dout.begin() == he - ho.begin());
  ASSERT_TRUE(same(thrust::host_vector<T>(dout.begin(), de), thrust::host_vector<T>(ho.begin(), he)));
  auto hr = thrust::partition_copy(h.begin(), h.end(), ho.begin(), hf.begin(), pred);
  auto dr = thrust::partition_copy(d.begin(), d.end(), dout.begin(), dfalse.begin(), pred);
  ASSERT_TRUE(dr.first - dout.begin() == hr.first - ho.begin() && dr.second - dfalse.begin() == hr.second - hf.begin());
  ASSERT_TRUE(same(thrust::host_vector<T>(dout.begin(), dr.first), thrust::host_vector<T>(ho.begin(), hr.first)));
  ASSERT_TRUE(same(thrust::host_vector<T>(dfalse.begin(), dr.second), thrust::host_vector<T>(hf.begin(), hr.second)));
  thrust::host_vector<T> hp(h);
  thrust::device_vector<T> dp(d);
  auto hm = thrust::stable_partition(hp.begin(), hp.end(), pred);
  auto dm = thrust::stable_partition(dp.begin(), dp.end(), pred);
  ASSERT_TRUE(dm - dp.begin() == hm - hp.begin());
  ASSERT_TRUE(same(to_host(dp), hp));
  hp = h;
  dp = d;
  auto hend = thrust::remove_if(hp.begin(), hp.end(), pred);
  auto dend = thrust::remove_if(dp.begin(), dp.end(), pred);
  ASSERT_TRUE(dend - dp.begin() == hend - hp.begin());
  ASSERT_TRUE(same(thrust::host_vector<T>(dp.begin(), dend), thrust::host_vector<T>(hp.begin(), hend)));
}

static void TestUserPredicateSelectionShapes() {
  for (size_t n : {(size_t)1, (size_t)777, (size_t)40000, (size_t)300001, ((size_t)1 << 20) + 3}) {
    const thrust::host_vector<int> h = random_values<int>(n, 21, 1000);
    thrust::host_vector<point> hpnt(n);
    thrust::host_vector<quad> hq(n);
    thrust::host_vector<unsigned char> hb(n);
    thrust::host_vector<double> hd(n);
    thrust::host_vector<short> hsh(n);
    for (size_t i = 0; i < n; ++i) {
      hpnt[i].x = (int)(mix(i + 5) % 1000);
      hpnt[i].w = (float)i;
      hq[i] = quad{(int)(mix(i) % 250), (int)(mix(i + 1) % 250), (int)(mix(i + 2) % 250), (int)(mix(i + 3) % 250)};
      hb[i] = (unsigned char)(mix(i + 9) % 256);
      hd[i] = (double)(mix(i + 11) % 1000) / 7.0;
      hsh[i] = (short)(mix(i + 13) % 1000);
    }
    for (int limit : {0, 30, 500, 970, 1000}) {
      g_test = "selection with a user predicate on the elements";
      CheckSelectionOnTheElements(h, below{limit});
      CheckSelectionOnTheElements(hpnt, point_below{limit});
      g_test = "selection with a user predicate on a stencil";
      CheckSelectionForms(hpnt, h, below{limit});          // 8-byte items, 4-byte stencil
      CheckSelectionForms(hsh, hq, quad_sum_below{limit});  // 2-byte items, 16-byte stencil
      CheckSelectionForms(hd, hpnt, point_below{limit});    // 8-byte items, 8-byte struct stencil
    }
    g_test = "selection with stencils of one and eight bytes";
    CheckSelectionForms(h, hb, byte_is_odd());
    CheckSelectionForms(hb, hd, double_below{40.0});
    g_test = "unique on structs with a user equality";
    {
      thrust::host_vector<point> hs2(hpnt);
      for (size_t i = 0; i < n; ++i) hs2[i].x = (int)(i / 3 + mix(i / 5) % 3);
      thrust::device_vector<point> ds2(hs2), dout(n);
      thrust::host_vector<point> hout(n);
      auto he = thrust::unique_copy(hs2.begin(), hs2.end(), hout.begin(), same_point_x());
      auto de = thrust::unique_copy(ds2.begin(), ds2.end(), dout.begin(), same_point_x());
      ASSERT_TRUE(de - dout.begin() == he - hout.begin());
      ASSERT_TRUE(same(thrust::host_vector<point>(dout.begin(), de), thrust::host_vector<point>(hout.begin(), he)));
      thrust::host_vector<short> hv(hsh), hvo(n);
      thrust::device_vector<short> dv(hsh), dvo(n);
      auto hu = thrust::unique_by_key_copy(hs2.begin(), hs2.end(), hv.begin(), hout.begin(), hvo.begin(), same_point_x());
      auto du = thrust::unique_by_key_copy(ds2.begin(), ds2.end(), dv.begin(), dout.begin(), dvo.begin(), same_point_x());
      ASSERT_TRUE(du.first - dout.begin() == hu.first - hout.begin());
      ASSERT_TRUE(same(thrust::host_vector<point>(dout.begin(), du.first), thrust::host_vector<point>(hout.begin(), hu.first)));
      ASSERT_TRUE(same(thrust::host_vector<short>(dvo.begin(), du.second), thrust::host_vector<short>(hvo.begin(), hu.second)));
      auto hin = thrust::unique(hs2.begin(), hs2.end(), same_point_x());
      auto din = thrust::unique(ds2.begin(), ds2.end(), same_point_x());
      ASSERT_TRUE(din - ds2.begin() == hin - hs2.begin());
      ASSERT_TRUE(same(thrust::host_vector<point>(ds2.begin(), din), thrust::host_vector<point>(hs2.begin(), hin)));
    }
  }
}

int main() {
  TestKnownAnswers();
  TestReduceWithBigIndexes();
  TestScanAndCopyWithBigIndexes();
  TestDiscardAndForeignOperator();
  TestAsyncForEachTransformWhenAll();
  Differential();
  TestUserPredicateSelectionShapes();
  TestUserOperators();
  TestUserOperatorScansOfLargeRanges();
  TestWideElements();
  TestUserPredicatesByKey();
  TestReduceByKeyWithUserFunctors();
  TestZipIterator();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
