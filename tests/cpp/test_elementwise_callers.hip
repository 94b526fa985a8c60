// Front-end test compiled with hipcc: the element-wise callers around the path and the checks
// that go with sort and partition: is_sorted / is_sorted_until, is_partitioned / partition_point,
// adjacent_difference, replace / replace_if / replace_copy(_if) with and without stencils,
// generate(_n), tabulate, reverse(_copy), swap_ranges, uninitialized_fill(_n), uninitialized_copy(_n).
// Literal vectors of the reference's unit tests (testing/is_sorted.cu:6-60, is_sorted_until.cu:6-60,
// partition_point.cu:6-40, is_partitioned.cu:6-60, adjacent_difference.cu:6-60, replace.cu:6-260,
// generate.cu:20-80, tabulate.cu:6-60, reverse.cu:6-60, swap_ranges.cu:6-40, uninitialized_fill.cu:6-60,
// uninitialized_copy.cu) on host_vector and device_vector, then device against host on random inputs.
#include <thrust/adjacent_difference.h>
#include <thrust/device_vector.h>
#include <thrust/functional.h>
#include <thrust/generate.h>
#include <thrust/host_vector.h>
#include <thrust/partition.h>
#include <thrust/replace.h>
#include <thrust/reverse.h>
#include <thrust/sequence.h>
#include <thrust/sort.h>
#include <thrust/swap.h>
#include <thrust/tabulate.h>
#include <thrust/uninitialized_copy.h>
#include <thrust/uninitialized_fill.h>

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
template <typename Vector, typename T>
static bool holds(const Vector& v, std::initializer_list<T> want) {
  if (v.size() != want.size()) return false;
  size_t i = 0;
  for (T w : want)
    if (!(v[i++] == (typename Vector::value_type)w)) return false;
  return true;
}
static const size_t kSizes[] = {0, 1, 2, 3, 63, 64, 65, 1000, 4097, 100000, (1u << 20) + 7};

template <typename T>
struct less_than_five {
  __host__ __device__ bool operator()(const T& v) const { return v < T(5); }
};
template <typename T>
struct return_value {
  T value;
  __host__ __device__ T operator()() const { return value; }
};
template <typename T>
struct cube_of_index {
  __host__ __device__ T operator()(std::ptrdiff_t i) const { return (T)(i * i * i); }
};
template <typename T>
struct negated_index {
  __host__ __device__ T operator()(std::ptrdiff_t i) const { return (T)(-(long long)i); }
};

template <typename Vector>
static void IsSorted() {
  typedef typename Vector::value_type T;
  g_test = "is_sorted / is_sorted_until: literal vectors";
  Vector v(4);
  v[0] = 0; v[1] = 5; v[2] = 8; v[3] = 0;
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.begin() + 0), true);
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.begin() + 1), true);
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.begin() + 2), true);
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.begin() + 3), true);
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.begin() + 4), false);
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.begin() + 3, thrust::less<T>()), true);
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.begin() + 1, thrust::greater<T>()), true);
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.begin() + 4, thrust::greater<T>()), false);
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.end()), false);
  ASSERT_EQUAL(thrust::is_sorted_until(v.begin(), v.end()) - v.begin(), 3);
  ASSERT_EQUAL(thrust::is_sorted_until(v.begin(), v.begin() + 3) - v.begin(), 3);
  ASSERT_EQUAL(thrust::is_sorted_until(v.begin(), v.begin() + 1) - v.begin(), 1);
  ASSERT_EQUAL(thrust::is_sorted_until(v.begin(), v.begin() + 0) - v.begin(), 0);
  ASSERT_EQUAL(thrust::is_sorted_until(v.begin(), v.end(), thrust::greater<T>()) - v.begin(), 1);
  v[0] = 1; v[1] = 1; v[2] = 1; v[3] = 1;  // equal elements are sorted under both orders
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.end()), true);
  ASSERT_EQUAL(thrust::is_sorted(v.begin(), v.end(), thrust::greater<T>()), true);
  Vector big(100000);
  thrust::sequence(big.begin(), big.end());
  ASSERT_EQUAL(thrust::is_sorted(big.begin(), big.end()), true);
  ASSERT_EQUAL(thrust::is_sorted_until(big.begin(), big.end()) - big.begin(), 100000);
  big[77777] = 0;
  ASSERT_EQUAL(thrust::is_sorted(big.begin(), big.end()), false);
  ASSERT_EQUAL(thrust::is_sorted_until(big.begin(), big.end()) - big.begin(), 77777);
  big[99] = 0;  // the first break counts
  ASSERT_EQUAL(thrust::is_sorted_until(big.begin(), big.end()) - big.begin(), 99);
}

template <typename Vector>
static void PartitionPoint() {
  typedef typename Vector::value_type T;
  g_test = "partition_point / is_partitioned: literal vectors";
  Vector v(4);
  v[0] = 1; v[1] = 1; v[2] = 1; v[3] = 0;
  ASSERT_EQUAL(thrust::partition_point(v.begin(), v.end(), thrust::identity<T>()) - v.begin(), 3);
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.end(), thrust::identity<T>()), true);
  v[2] = 0;
  ASSERT_EQUAL(thrust::partition_point(v.begin(), v.end(), thrust::identity<T>()) - v.begin(), 2);
  v[0] = 0; v[1] = 0;
  ASSERT_EQUAL(thrust::partition_point(v.begin(), v.end(), thrust::identity<T>()) - v.begin(), 0);
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.end(), thrust::identity<T>()), true);
  v[0] = 1; v[1] = 1; v[2] = 1; v[3] = 1;
  ASSERT_EQUAL(thrust::partition_point(v.begin(), v.end(), thrust::identity<T>()) - v.begin(), 4);
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.end(), thrust::identity<T>()), true);
  v[0] = 1; v[1] = 1; v[2] = 0; v[3] = 0;
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.begin() + 0, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.begin() + 1, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.begin() + 2, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.begin() + 3, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.begin() + 4, thrust::identity<T>()), true);
  v[0] = 1; v[1] = 0; v[2] = 1; v[3] = 0;
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.begin() + 2, thrust::identity<T>()), true);
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.begin() + 3, thrust::identity<T>()), false);
  ASSERT_EQUAL(thrust::is_partitioned(v.begin(), v.begin() + 4, thrust::identity<T>()), false);
  // a partition made by thrust::partition is one, and its point is the returned iterator
  thrust::host_vector<T> h = samples<T>(50000, 3, 10);
  Vector data = h;
  auto mid = thrust::stable_partition(data.begin(), data.end(), less_than_five<T>());
  ASSERT_EQUAL(thrust::is_partitioned(data.begin(), data.end(), less_than_five<T>()), true);
  ASSERT_TRUE(thrust::partition_point(data.begin(), data.end(), less_than_five<T>()) == mid);
  data[data.size() - 1] = 0;  // one element that passes, behind the point
  ASSERT_EQUAL(thrust::is_partitioned(data.begin(), data.end(), less_than_five<T>()), false);
}

template <typename Vector>
static void AdjacentDifference() {
  typedef typename Vector::value_type T;
  g_test = "adjacent_difference: literal vectors";
  Vector input(3), output(3);
  input[0] = 1; input[1] = 4; input[2] = 6;
  auto end = thrust::adjacent_difference(input.begin(), input.end(), output.begin());
  ASSERT_EQUAL(end - output.begin(), 3);
  ASSERT_TRUE(holds(output, {1, 3, 2}));
  end = thrust::adjacent_difference(input.begin(), input.end(), output.begin(), thrust::plus<T>());
  ASSERT_EQUAL(end - output.begin(), 3);
  ASSERT_TRUE(holds(output, {1, 5, 10}));
  // in place
  thrust::adjacent_difference(input.begin(), input.end(), input.begin(), thrust::plus<T>());
  ASSERT_TRUE(holds(input, {1, 5, 10}));
  Vector none(0);
  ASSERT_TRUE(thrust::adjacent_difference(none.begin(), none.end(), none.begin()) == none.begin());
}

template <typename T>
static void AdjacentDifferenceAgainstHost() {
  g_test = "adjacent_difference: device against host";
  for (size_t n : kSizes) {
    thrust::host_vector<T> h = samples<T>(n, 41 + n, 1000), ho(n);
    thrust::device_vector<T> d = h, dout(n);
    thrust::adjacent_difference(h.begin(), h.end(), ho.begin());
    thrust::adjacent_difference(d.begin(), d.end(), dout.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
    thrust::adjacent_difference(d.begin(), d.end(), d.begin());  // in place
    ASSERT_TRUE(same(thrust::host_vector<T>(d), ho));
    thrust::adjacent_difference(h.begin(), h.end(), h.begin());
    ASSERT_TRUE(same(h, ho));
    // in place through iterators of different types: a const and a plain iterator of one vector, a raw
    // pointer and a device_ptr of one array
    thrust::device_vector<T> d2 = samples<T>(n, 41 + n, 1000);
    thrust::adjacent_difference(d2.cbegin(), d2.cend(), d2.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(d2), ho));
    thrust::device_vector<T> d3 = samples<T>(n, 41 + n, 1000);
    if (n > 0) {
      const T* raw = thrust::raw_pointer_cast(d3.data());
      thrust::adjacent_difference(thrust::device, raw, raw + n, d3.data());
      ASSERT_TRUE(same(thrust::host_vector<T>(d3), ho));
    }
    // the differences of a scan give the input back
    thrust::host_vector<T> again(n);
    thrust::device_vector<T> scanned = ho;
    thrust::inclusive_scan(scanned.begin(), scanned.end(), scanned.begin());
    thrust::adjacent_difference(scanned.begin(), scanned.end(), scanned.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(scanned), ho));
  }
}

template <typename Vector>
static void Replace() {
  typedef typename Vector::value_type T;
  g_test = "replace family: literal vectors";
  Vector data(5);
  data[0] = 1; data[1] = 2; data[2] = 1; data[3] = 3; data[4] = 2;
  thrust::replace(data.begin(), data.end(), (T)1, (T)4);
  thrust::replace(data.begin(), data.end(), (T)2, (T)5);
  ASSERT_TRUE(holds(data, {4, 5, 4, 3, 5}));
  data[0] = 1; data[1] = 2; data[2] = 1; data[3] = 3; data[4] = 2;
  Vector dest(5);
  auto end = thrust::replace_copy(data.begin(), data.end(), dest.begin(), (T)1, (T)4);
  ASSERT_EQUAL(end - dest.begin(), 5);
  thrust::replace_copy(dest.begin(), dest.end(), dest.begin(), (T)2, (T)5);
  ASSERT_TRUE(holds(dest, {4, 5, 4, 3, 5}));
  ASSERT_TRUE(holds(data, {1, 2, 1, 3, 2}));
  data[0] = 1; data[1] = 3; data[2] = 4; data[3] = 6; data[4] = 5;
  thrust::replace_if(data.begin(), data.end(), less_than_five<T>(), (T)0);
  ASSERT_TRUE(holds(data, {0, 0, 0, 6, 5}));
  data[0] = 1; data[1] = 3; data[2] = 4; data[3] = 6; data[4] = 5;
  Vector stencil(5);
  stencil[0] = 5; stencil[1] = 4; stencil[2] = 6; stencil[3] = 3; stencil[4] = 7;
  thrust::replace_if(data.begin(), data.end(), stencil.begin(), less_than_five<T>(), (T)0);
  ASSERT_TRUE(holds(data, {1, 0, 4, 0, 5}));
  data[0] = 1; data[1] = 3; data[2] = 4; data[3] = 6; data[4] = 5;
  end = thrust::replace_copy_if(data.begin(), data.end(), dest.begin(), less_than_five<T>(), (T)0);
  ASSERT_EQUAL(end - dest.begin(), 5);
  ASSERT_TRUE(holds(dest, {0, 0, 0, 6, 5}));
  end = thrust::replace_copy_if(data.begin(), data.end(), stencil.begin(), dest.begin(), less_than_five<T>(), (T)0);
  ASSERT_EQUAL(end - dest.begin(), 5);
  ASSERT_TRUE(holds(dest, {1, 0, 4, 0, 5}));
  ASSERT_TRUE(holds(data, {1, 3, 4, 6, 5}));
}

template <typename T>
static void ReplaceAgainstHost() {
  g_test = "replace family: device against host";
  for (size_t n : kSizes) {
    thrust::host_vector<T> h = samples<T>(n, 51 + n, 10), hs = samples<T>(n, 52 + n, 10), ho(n);
    thrust::device_vector<T> d = h, ds = hs, dout(n);
    thrust::replace_copy(h.begin(), h.end(), ho.begin(), (T)3, (T)77);
    thrust::replace_copy(d.begin(), d.end(), dout.begin(), (T)3, (T)77);
    ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
    thrust::replace_copy_if(h.begin(), h.end(), hs.begin(), ho.begin(), less_than_five<T>(), (T)88);
    thrust::replace_copy_if(d.begin(), d.end(), ds.begin(), dout.begin(), less_than_five<T>(), (T)88);
    ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
    thrust::replace_if(h.begin(), h.end(), less_than_five<T>(), (T)9);
    thrust::replace_if(d.begin(), d.end(), less_than_five<T>(), (T)9);
    ASSERT_TRUE(same(thrust::host_vector<T>(d), h));
  }
}

template <typename Vector>
static void GenerateTabulateReverseSwap() {
  typedef typename Vector::value_type T;
  g_test = "generate / tabulate / reverse / swap_ranges / uninitialized_*: literal vectors";
  Vector v(5, T(0));
  const return_value<T> thirteen = {T(13)};
  thrust::generate(v.begin(), v.end(), thirteen);
  ASSERT_TRUE(holds(v, {13, 13, 13, 13, 13}));
  const return_value<T> seven = {T(7)};
  auto gend = thrust::generate_n(v.begin() + 1, 3, seven);
  ASSERT_EQUAL(gend - v.begin(), 4);
  ASSERT_TRUE(holds(v, {13, 7, 7, 7, 13}));

  thrust::tabulate(v.begin(), v.end(), thrust::identity<T>());
  ASSERT_TRUE(holds(v, {0, 1, 2, 3, 4}));
  thrust::tabulate(v.begin(), v.end(), negated_index<T>());
  ASSERT_TRUE(holds(v, {0, -1, -2, -3, -4}));
  thrust::tabulate(v.begin(), v.end(), cube_of_index<T>());
  ASSERT_TRUE(holds(v, {0, 1, 8, 27, 64}));

  v[0] = 1; v[1] = 2; v[2] = 3; v[3] = 4; v[4] = 5;
  thrust::reverse(v.begin(), v.end());
  ASSERT_TRUE(holds(v, {5, 4, 3, 2, 1}));
  Vector out(5, T(0));
  auto rend = thrust::reverse_copy(v.begin(), v.end(), out.begin());
  ASSERT_EQUAL(rend - out.begin(), 5);
  ASSERT_TRUE(holds(out, {1, 2, 3, 4, 5}));
  ASSERT_TRUE(holds(v, {5, 4, 3, 2, 1}));
  thrust::reverse(v.begin(), v.begin() + 4);  // an even count
  ASSERT_TRUE(holds(v, {2, 3, 4, 5, 1}));
  thrust::reverse(v.begin(), v.begin() + 1);
  thrust::reverse(v.begin(), v.begin());
  ASSERT_TRUE(holds(v, {2, 3, 4, 5, 1}));

  Vector v1(5), v2(5);
  for (int i = 0; i < 5; ++i) { v1[i] = T(i); v2[i] = T(5 + i); }
  auto send = thrust::swap_ranges(v1.begin(), v1.end(), v2.begin());
  ASSERT_EQUAL(send - v2.begin(), 5);
  ASSERT_TRUE(holds(v1, {5, 6, 7, 8, 9}));
  ASSERT_TRUE(holds(v2, {0, 1, 2, 3, 4}));

  Vector u(5, T(0));
  thrust::uninitialized_fill(u.begin() + 1, u.begin() + 4, T(7));
  ASSERT_TRUE(holds(u, {0, 7, 7, 7, 0}));
  auto uend = thrust::uninitialized_fill_n(u.begin(), 2, T(8));
  ASSERT_EQUAL(uend - u.begin(), 2);
  ASSERT_TRUE(holds(u, {8, 8, 7, 7, 0}));
  Vector w(5, T(0));
  auto cend = thrust::uninitialized_copy(u.begin(), u.end(), w.begin());
  ASSERT_EQUAL(cend - w.begin(), 5);
  ASSERT_TRUE(holds(w, {8, 8, 7, 7, 0}));
  cend = thrust::uninitialized_copy_n(v1.begin(), 3, w.begin());
  ASSERT_EQUAL(cend - w.begin(), 3);
  ASSERT_TRUE(holds(w, {5, 6, 7, 7, 0}));
}

template <typename T>
static void ReverseAndSwapAgainstHost() {
  g_test = "reverse / swap_ranges / tabulate: device against host";
  for (size_t n : kSizes) {
    thrust::host_vector<T> h = samples<T>(n, 61 + n, 1000), h2 = samples<T>(n, 62 + n, 1000), ho(n);
    thrust::device_vector<T> d = h, d2 = h2, dout(n);
    thrust::reverse_copy(h.begin(), h.end(), ho.begin());
    thrust::reverse_copy(d.begin(), d.end(), dout.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
    thrust::reverse(d.begin(), d.end());
    ASSERT_TRUE(same(thrust::host_vector<T>(d), ho));
    thrust::reverse(d.begin(), d.end());
    ASSERT_TRUE(same(thrust::host_vector<T>(d), h));
    thrust::swap_ranges(d.begin(), d.end(), d2.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(d), h2));
    ASSERT_TRUE(same(thrust::host_vector<T>(d2), h));
    thrust::tabulate(h.begin(), h.end(), cube_of_index<T>());
    thrust::tabulate(d.begin(), d.end(), cube_of_index<T>());
    ASSERT_TRUE(same(thrust::host_vector<T>(d), h));
  }
}

template <typename T>
static void IsSortedAgainstHost() {
  g_test = "is_sorted_until: device against host";
  for (size_t n : kSizes) {
    thrust::host_vector<T> h = samples<T>(n, 71 + n, 1000);
    thrust::device_vector<T> d = h;
    ASSERT_EQUAL(thrust::is_sorted_until(d.begin(), d.end()) - d.begin(), thrust::is_sorted_until(h.begin(), h.end()) - h.begin());
    thrust::sort(d.begin(), d.end());
    ASSERT_EQUAL(thrust::is_sorted(d.begin(), d.end()), true);
    ASSERT_EQUAL(thrust::is_sorted(d.begin(), d.end(), thrust::greater<T>()), n < 2 || d[0] == d[n - 1]);
    thrust::sort(d.begin(), d.end(), thrust::greater<T>());
    ASSERT_EQUAL(thrust::is_sorted(d.begin(), d.end(), thrust::greater<T>()), true);
  }
}

struct adds_one_in_place {
  template <typename T>
  __host__ __device__ void operator()(T& x) const { x = x + T(1); }
};
struct times_three_plus_one {
  template <typename T>
  __host__ __device__ T operator()(const T& x) const { return (T)(x * 3 + 1); }
};
struct widens {
  __host__ __device__ long long operator()(int x) const { return (long long)x * 1000000007ll; }
};
struct bumps_and_doubles {  // changes its argument: the input must change too
  __host__ __device__ int operator()(int& x) const { x += 1; return 2 * x; }
};

struct position_writer {
  const int* base;
  __host__ __device__ void operator()(int& x) const { x = (int)(&x - base); }
};
struct position_reader {
  const int* base;
  __host__ __device__ int operator()(const int& x) const { return (int)(&x - base); }
};

// thrust::transform over plain arrays takes kernels that move 16 bytes per access when the arrays are
// aligned for it: sizes around the switch, tails, offsets that break the alignment, 8-byte and mixed
// element sizes, in place, and a functor that modifies its argument
template <typename T>
static void TransformShapes() {
  g_test = "transform: array shapes";
  const size_t sizes[] = {1, 3, 4095, 4096, 4097, 4099, 10001, 65536 + 3, (1u << 20) + 5};
  for (size_t n : sizes) {
    for (size_t offset : {size_t(0), size_t(1), size_t(2)}) {
      thrust::host_vector<T> h = samples<T>(n + offset, 101 + n, 1000), h2 = samples<T>(n + offset, 102 + n, 1000);
      thrust::host_vector<T> ho(n + offset, T(7));
      thrust::device_vector<T> d = h, d2 = h2, dout = ho;
      thrust::transform(h.begin() + offset, h.end(), ho.begin() + offset, times_three_plus_one());
      thrust::transform(d.begin() + offset, d.end(), dout.begin() + offset, times_three_plus_one());
      ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
      thrust::transform(h.begin() + offset, h.end(), h2.begin(), ho.begin() + offset, thrust::minus<T>());
      thrust::transform(d.begin() + offset, d.end(), d2.begin(), dout.begin() + offset, thrust::minus<T>());
      ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
      thrust::transform(h.begin(), h.end(), h.begin(), times_three_plus_one());  // in place
      thrust::transform(d.begin(), d.end(), d.begin(), times_three_plus_one());
      ASSERT_TRUE(same(thrust::host_vector<T>(d), h));
      thrust::adjacent_difference(h.begin() + offset, h.end(), ho.begin() + offset);
      thrust::adjacent_difference(d.begin() + offset, d.end(), dout.begin() + offset);
      ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
    }
  }
  for (size_t n : sizes) {
    for (size_t offset : {size_t(0), size_t(1)}) {
      thrust::host_vector<T> h = samples<T>(n + offset, 111 + n, 1000);
      thrust::device_vector<T> d = h;
      thrust::for_each(h.begin() + offset, h.end(), adds_one_in_place());
      thrust::for_each(d.begin() + offset, d.end(), adds_one_in_place());
      ASSERT_TRUE(same(thrust::host_vector<T>(d), h));
      thrust::generate(d.begin() + offset, d.end(), return_value<T>{T(5)});
      thrust::fill(h.begin() + offset, h.end(), T(5));
      ASSERT_TRUE(same(thrust::host_vector<T>(d), h));
    }
  }
  thrust::host_vector<int> hi = samples<int>(70001, 7, 100000);
  thrust::device_vector<int> di = hi;
  thrust::host_vector<long long> hw(hi.size());
  thrust::device_vector<long long> dw(hi.size());
  thrust::transform(hi.begin(), hi.end(), hw.begin(), widens());
  thrust::transform(di.begin(), di.end(), dw.begin(), widens());
  ASSERT_TRUE(same(thrust::host_vector<long long>(dw), hw));
  thrust::host_vector<int> hb(hi.size());
  thrust::device_vector<int> db(hi.size());
  thrust::transform(hi.begin(), hi.end(), hb.begin(), bumps_and_doubles());
  thrust::transform(di.begin(), di.end(), db.begin(), bumps_and_doubles());
  ASSERT_TRUE(same(thrust::host_vector<int>(db), hb));
  ASSERT_TRUE(same(thrust::host_vector<int>(di), hi));  // both inputs were bumped
  // the same functor with the output on the input: the results, not the bumped inputs, stay
  thrust::transform(hi.begin(), hi.end(), hi.begin(), bumps_and_doubles());
  thrust::transform(di.begin(), di.end(), di.begin(), bumps_and_doubles());
  ASSERT_TRUE(same(thrust::host_vector<int>(di), hi));
  // a functor is handed the element where it lies: its address gives the element's position
  // (thrust/system/cuda/detail/for_each.h:58), on aligned arrays of any size as well
  for (size_t n : {size_t(5), size_t(4096), size_t(70001)}) {
    thrust::device_vector<int> where(n, -1);
    const position_writer writes = {thrust::raw_pointer_cast(where.data())};
    thrust::for_each(where.begin(), where.end(), writes);
    thrust::host_vector<int> expect(n);
    thrust::sequence(expect.begin(), expect.end());
    ASSERT_TRUE(same(thrust::host_vector<int>(where), expect));
    thrust::device_vector<int> from(n, 3), positions(n);
    const position_reader reads = {thrust::raw_pointer_cast(from.data())};
    thrust::transform(from.begin(), from.end(), positions.begin(), reads);
    ASSERT_TRUE(same(thrust::host_vector<int>(positions), expect));
  }
}

int main() {
  TransformShapes<int>();
  TransformShapes<float>();
  TransformShapes<long long>();
  TransformShapes<double>();
  IsSorted<thrust::host_vector<int> >();
  IsSorted<thrust::device_vector<int> >();
  IsSorted<thrust::device_vector<float> >();
  IsSortedAgainstHost<int>();
  IsSortedAgainstHost<unsigned short>();
  PartitionPoint<thrust::host_vector<int> >();
  PartitionPoint<thrust::device_vector<int> >();
  PartitionPoint<thrust::device_vector<short> >();
  AdjacentDifference<thrust::host_vector<int> >();
  AdjacentDifference<thrust::device_vector<int> >();
  AdjacentDifference<thrust::device_vector<long long> >();
  AdjacentDifferenceAgainstHost<int>();
  AdjacentDifferenceAgainstHost<unsigned int>();
  Replace<thrust::host_vector<int> >();
  Replace<thrust::device_vector<int> >();
  Replace<thrust::device_vector<float> >();
  ReplaceAgainstHost<int>();
  ReplaceAgainstHost<short>();
  GenerateTabulateReverseSwap<thrust::host_vector<int> >();
  GenerateTabulateReverseSwap<thrust::device_vector<int> >();
  GenerateTabulateReverseSwap<thrust::device_vector<long long> >();
  GenerateTabulateReverseSwap<thrust::device_vector<float> >();
  ReverseAndSwapAgainstHost<int>();
  ReverseAndSwapAgainstHost<long long>();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
