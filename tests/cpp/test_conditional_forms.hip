// Front-end test compiled with hipcc: transform_if (three forms), gather_if, scatter_if, for_each_n
// and thrust::reverse_iterator.  Literal vectors of the reference's unit tests
// (testing/transform.cu:120-330, gather.cu:120-200, scatter.cu:110-200, for_each.cu:60-140,
// reverse_iterator.cu:6-90) on host_vector and device_vector, then device against host.
#include <thrust/copy.h>
#include <thrust/device_vector.h>
#include <thrust/functional.h>
#include <thrust/gather.h>
#include <thrust/host_vector.h>
#include <thrust/iterator/reverse_iterator.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/scatter.h>
#include <thrust/sequence.h>
#include <thrust/sort.h>
#include <thrust/transform.h>
#include <thrust/addressof.h>
#include <thrust/advance.h>
#include <thrust/device_delete.h>
#include <thrust/device_malloc_allocator.h>
#include <thrust/device_new.h>
#include <thrust/device_new_allocator.h>
#include <thrust/iterator/transform_output_iterator.h>
#include <thrust/limits.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/zip_function.h>

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
static const size_t kSizes[] = {0, 1, 2, 63, 64, 65, 1000, 4097, 100000, (1u << 20) + 7};

template <typename T>
struct is_even {
  __host__ __device__ bool operator()(const T& x) const { return ((long long)x & 1) == 0; }
};
template <typename T>
struct is_zero {
  __host__ __device__ bool operator()(const T& x) const { return x == T(0); }
};
template <typename T>
struct adds_ten {
  __host__ __device__ void operator()(T& x) const { x = x + T(10); }
};

template <typename Vector>
static void TransformIf() {
  typedef typename Vector::value_type T;
  g_test = "transform_if: literal vectors";
  Vector input(3), stencil(3), output(3);
  input[0] = 1; input[1] = -2; input[2] = 3;
  stencil[0] = 1; stencil[1] = 0; stencil[2] = 1;
  output[0] = 1; output[1] = 2; output[2] = 3;
  auto end = thrust::transform_if(input.begin(), input.end(), stencil.begin(), output.begin(), thrust::negate<T>(),
                                  thrust::identity<T>());
  ASSERT_EQUAL(end - output.begin(), 3);
  ASSERT_TRUE(holds(output, {-1, 2, -3}));
  // without a stencil the input decides
  input[0] = 0; input[1] = -2; input[2] = 0;
  output[0] = -1; output[1] = -2; output[2] = -3;
  end = thrust::transform_if(input.begin(), input.end(), output.begin(), thrust::negate<T>(), thrust::identity<T>());
  ASSERT_EQUAL(end - output.begin(), 3);
  ASSERT_TRUE(holds(output, {-1, 2, -3}));
  // two inputs, written where the stencil is zero
  Vector input2(3);
  input[0] = 1; input[1] = -2; input[2] = 3;
  input2[0] = -4; input2[1] = 5; input2[2] = 6;
  stencil[0] = 0; stencil[1] = 1; stencil[2] = 0;
  output[0] = 1; output[1] = 2; output[2] = 3;
  end = thrust::transform_if(input.begin(), input.end(), input2.begin(), stencil.begin(), output.begin(),
                             thrust::minus<T>(), is_zero<T>());
  ASSERT_EQUAL(end - output.begin(), 3);
  ASSERT_TRUE(holds(output, {5, 2, -3}));
}

template <typename Vector, typename IntVector>
static void GatherScatterIf() {
  g_test = "gather_if / scatter_if: literal vectors";
  IntVector flg(5), map(5);
  Vector src(8), dst(5, 0);
  flg[0] = 0; flg[1] = 1; flg[2] = 0; flg[3] = 1; flg[4] = 0;
  map[0] = 6; map[1] = 2; map[2] = 1; map[3] = 7; map[4] = 2;
  for (int i = 0; i < 8; ++i) src[i] = i;
  auto end = thrust::gather_if(map.begin(), map.end(), flg.begin(), src.begin(), dst.begin());
  ASSERT_EQUAL(end - dst.begin(), 5);
  ASSERT_TRUE(holds(dst, {0, 2, 0, 7, 0}));
  thrust::gather_if(map.begin(), map.end(), flg.begin(), src.begin(), dst.begin(), is_even<int>());  // where the flag is 0
  ASSERT_TRUE(holds(dst, {6, 2, 1, 7, 2}));

  Vector from(5), to(8, 0);
  map[0] = 6; map[1] = 3; map[2] = 1; map[3] = 7; map[4] = 2;
  for (int i = 0; i < 5; ++i) from[i] = i;
  thrust::scatter_if(from.begin(), from.end(), map.begin(), flg.begin(), to.begin());
  ASSERT_TRUE(holds(to, {0, 0, 0, 1, 0, 0, 0, 3}));
  thrust::scatter_if(from.begin(), from.end(), map.begin(), flg.begin(), to.begin(), is_even<int>());
  ASSERT_TRUE(holds(to, {0, 2, 4, 1, 0, 0, 0, 3}));
}

template <typename Vector>
static void ForEachN() {
  typedef typename Vector::value_type T;
  g_test = "for_each_n";
  Vector v(5);
  for (int i = 0; i < 5; ++i) v[i] = T(i);
  auto end = thrust::for_each_n(v.begin(), 3, adds_ten<T>());
  ASSERT_EQUAL(end - v.begin(), 3);
  ASSERT_TRUE(holds(v, {10, 11, 12, 3, 4}));
  end = thrust::for_each_n(v.begin(), 0, adds_ten<T>());
  ASSERT_EQUAL(end - v.begin(), 0);
  ASSERT_TRUE(holds(v, {10, 11, 12, 3, 4}));
}

template <typename Vector>
static void ReverseIterator() {
  typedef typename Vector::value_type T;
  g_test = "reverse_iterator";
  Vector v(4);
  v[0] = 3; v[1] = 4; v[2] = 5; v[3] = 6;
  thrust::reverse_iterator<typename Vector::iterator> rbegin(v.end()), rend(v.begin());
  ASSERT_EQUAL(rend - rbegin, 4);
  ASSERT_EQUAL((T)*rbegin, T(6));
  ASSERT_EQUAL((T)rbegin[1], T(5));
  ASSERT_EQUAL((T)*(rbegin + 3), T(3));
  ASSERT_TRUE(rbegin.base() == v.end());
  ASSERT_TRUE(thrust::make_reverse_iterator(v.end()) == rbegin);
  // read through it
  Vector out(4);
  thrust::copy(rbegin, rend, out.begin());
  ASSERT_TRUE(holds(out, {6, 5, 4, 3}));
  ASSERT_EQUAL(thrust::reduce(rbegin, rend), T(18));
  // write through it
  thrust::copy(v.begin(), v.end(), thrust::make_reverse_iterator(out.end()));
  ASSERT_TRUE(holds(out, {6, 5, 4, 3}));
  out[0] = 1; out[1] = 2; out[2] = 3; out[3] = 4;
  thrust::transform(out.begin(), out.end(), thrust::make_reverse_iterator(v.end()), thrust::negate<T>());
  ASSERT_TRUE(holds(v, {-4, -3, -2, -1}));
  // a scan from the right: the suffix sums
  v[0] = 1; v[1] = 2; v[2] = 3; v[3] = 4;
  thrust::inclusive_scan(thrust::make_reverse_iterator(v.end()), thrust::make_reverse_iterator(v.begin()),
                         thrust::make_reverse_iterator(out.end()));
  ASSERT_TRUE(holds(out, {10, 9, 7, 4}));
  // reversing twice gives the range back
  auto twice = thrust::make_reverse_iterator(thrust::make_reverse_iterator(v.begin()));
  ASSERT_EQUAL((T)*twice, T(1));
  ASSERT_EQUAL((T)twice[3], T(4));
}

struct sum_and_difference {
  template <typename T>
  __host__ __device__ void operator()(const T& a, const T& b, T& sum, T& difference) const {
    sum = a + b;
    difference = a - b;
  }
};
struct multiply_add {
  template <typename T>
  __host__ __device__ T operator()(const T& a, const T& b, const T& c) const { return a * b + c; }
};

template <typename Vector>
static void ZipFunctionAndAdvance() {
  typedef typename Vector::value_type T;
  g_test = "zip_function / advance";
  Vector a(4), b(4), c(4), sum(4), difference(4), out(4);
  for (int i = 0; i < 4; ++i) { a[i] = T(10 * i); b[i] = T(i + 1); c[i] = T(100); }
  // testing/zip_function.cu: a function of the elements applied to the zipped ranges
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(a.begin(), b.begin(), c.begin()));
  thrust::transform(zipped, zipped + 4, out.begin(), thrust::make_zip_function(multiply_add()));
  ASSERT_TRUE(holds(out, {100, 120, 160, 220}));
  auto four = thrust::make_zip_iterator(thrust::make_tuple(a.begin(), b.begin(), sum.begin(), difference.begin()));
  thrust::for_each(four, four + 4, thrust::make_zip_function(sum_and_difference()));
  ASSERT_TRUE(holds(sum, {1, 12, 23, 34}));
  ASSERT_TRUE(holds(difference, {-1, 8, 17, 26}));
  auto it = a.begin();
  thrust::advance(it, 3);
  ASSERT_EQUAL(it - a.begin(), 3);
  thrust::advance(it, -2);
  ASSERT_EQUAL((T)*it, T(10));
}

struct doubles {
  template <typename T>
  __host__ __device__ T operator()(const T& x) const { return x + x; }
};

template <typename Vector>
static void TransformOutputIterator() {
  typedef typename Vector::value_type T;
  g_test = "transform_output_iterator";
  // testing/transform_output_iterator.cu: what is written arrives transformed
  Vector input(4), output(4, T(0));
  for (int i = 0; i < 4; ++i) input[i] = T(i + 1);
  auto doubled = thrust::make_transform_output_iterator(output.begin(), doubles());
  thrust::copy(input.begin(), input.end(), doubled);
  ASSERT_TRUE(holds(output, {2, 4, 6, 8}));
  thrust::transform(input.begin(), input.end(), doubled, thrust::negate<T>());
  ASSERT_TRUE(holds(output, {-2, -4, -6, -8}));
  thrust::inclusive_scan(input.begin(), input.end(), doubled);
  ASSERT_TRUE(holds(output, {2, 6, 12, 20}));
  ASSERT_EQUAL((doubled + 3) - doubled, 3);
}

static void DeviceNewAndAllocators() {
  g_test = "device_new / device_delete / allocators";
  thrust::device_ptr<int> p = thrust::device_new<int>(5);
  for (int i = 0; i < 5; ++i) ASSERT_EQUAL((int)p[i], 0);
  p[2] = 7;
  ASSERT_EQUAL(thrust::reduce(p, p + 5), 7);
  thrust::device_delete(p, 5);
  thrust::device_ptr<void> raw = thrust::device_malloc(4 * sizeof(float));
  thrust::device_ptr<float> q = thrust::device_new<float>(raw, 2.5f, 4);
  ASSERT_EQUAL(thrust::reduce(q, q + 4), 10.0f);
  thrust::device_delete(q, 4);
  thrust::device_vector<int, thrust::device_malloc_allocator<int> > a(100, 3);
  ASSERT_EQUAL(thrust::reduce(a.begin(), a.end()), 300);
  thrust::device_vector<int, thrust::device_new_allocator<int> > b(50, 2);
  b.resize(80, 1);
  ASSERT_EQUAL(thrust::reduce(b.begin(), b.end()), 130);
  int on_host = 4;
  ASSERT_TRUE(thrust::addressof(on_host) == &on_host);
  ASSERT_EQUAL(thrust::numeric_limits<int>::max(), std::numeric_limits<int>::max());
}

template <typename T>
static void AgainstHost() {
  g_test = "conditional forms: device against host";
  for (size_t n : kSizes) {
    thrust::host_vector<T> h = samples<T>(n, 91 + n, 1000), h2 = samples<T>(n, 92 + n, 1000), ho = samples<T>(n, 93 + n, 7);
    thrust::host_vector<int> hs = samples<int>(n, 94 + n, 3);
    thrust::device_vector<T> d = h, d2 = h2, dout = ho;
    thrust::device_vector<int> ds = hs;
    thrust::transform_if(h.begin(), h.end(), h2.begin(), hs.begin(), ho.begin(), thrust::plus<T>(), is_even<int>());
    thrust::transform_if(d.begin(), d.end(), d2.begin(), ds.begin(), dout.begin(), thrust::plus<T>(), is_even<int>());
    ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
    thrust::transform_if(h.begin(), h.end(), ho.begin(), thrust::negate<T>(), is_even<T>());
    thrust::transform_if(d.begin(), d.end(), dout.begin(), thrust::negate<T>(), is_even<T>());
    ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
    // a random permutation as the map: sort positions by random keys
    thrust::host_vector<int> hmap(n);
    thrust::sequence(hmap.begin(), hmap.end());
    thrust::host_vector<unsigned> keys = samples<unsigned>(n, 95 + n, 1u << 30);
    thrust::sort_by_key(keys.begin(), keys.end(), hmap.begin());
    thrust::device_vector<int> dmap = hmap;
    thrust::gather_if(hmap.begin(), hmap.end(), hs.begin(), h.begin(), ho.begin());
    thrust::gather_if(dmap.begin(), dmap.end(), ds.begin(), d.begin(), dout.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
    thrust::scatter_if(h2.begin(), h2.end(), hmap.begin(), hs.begin(), ho.begin());
    thrust::scatter_if(d2.begin(), d2.end(), dmap.begin(), ds.begin(), dout.begin());
    ASSERT_TRUE(same(thrust::host_vector<T>(dout), ho));
    // sorting a reversed view descending sorts the range ascending from the back
    thrust::sort(thrust::make_reverse_iterator(d.end()), thrust::make_reverse_iterator(d.begin()));
    thrust::sort(h.begin(), h.end(), thrust::greater<T>());
    ASSERT_TRUE(same(thrust::host_vector<T>(d), h));
  }
}

int main() {
  TransformIf<thrust::host_vector<int> >();
  TransformIf<thrust::device_vector<int> >();
  TransformIf<thrust::device_vector<float> >();
  GatherScatterIf<thrust::host_vector<int>, thrust::host_vector<int> >();
  GatherScatterIf<thrust::device_vector<int>, thrust::device_vector<int> >();
  GatherScatterIf<thrust::device_vector<float>, thrust::device_vector<int> >();
  ForEachN<thrust::host_vector<int> >();
  ForEachN<thrust::device_vector<int> >();
  ForEachN<thrust::device_vector<double> >();
  ReverseIterator<thrust::host_vector<int> >();
  ReverseIterator<thrust::device_vector<int> >();
  ReverseIterator<thrust::device_vector<long long> >();
  ZipFunctionAndAdvance<thrust::host_vector<int> >();
  ZipFunctionAndAdvance<thrust::device_vector<int> >();
  ZipFunctionAndAdvance<thrust::device_vector<float> >();
  TransformOutputIterator<thrust::host_vector<int> >();
  TransformOutputIterator<thrust::device_vector<int> >();
  TransformOutputIterator<thrust::device_vector<double> >();
  DeviceNewAndAllocators();
  AgainstHost<int>();
  AgainstHost<long long>();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
