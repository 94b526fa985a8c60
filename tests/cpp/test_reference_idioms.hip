// Front-end test compiled with hipcc: the idioms the reference's example programs and unit tests
// lean on beside the algorithms themselves.  thrust::min / thrust::max and their tie rule
// (testing/min_and_max.cu:6-75), thrust::distance (testing/distance.cu:7-30), the storage calls of
// thrust/memory.h (testing/memory.cu:167-205), transform_input_output_iterator
// (testing/transform_input_output_iterator.cu:10-95), transform_iterator with a named value type,
// counting_iterator with a named system, device_vector iterators dereferenced inside a functor
// (raw_reference_cast), fill through a strided view, predicates that are not const-callable,
// unique over tuples, allocators over run-time chosen resources (thrust/mr/polymorphic_adaptor.h),
// iterators of the caller's own built on iterator_adaptor / iterator_facade, allocate_unique and
// device_make_unique, and what the vector
// headers bring along.
#include <thrust/device_vector.h>
#include <thrust/host_vector.h>
// (nothing else before the first test on purpose: fill, copy, reduce, distance and equal are reached
// through the vector headers, as programs written for the reference expect)

static int g_failed = 0, g_checks = 0;
static const char* g_test = "";
#include <cstdio>
#define ASSERT_TRUE(c)                                                                    \
  do {                                                                                    \
    ++g_checks;                                                                           \
    if (!(c)) { ++g_failed; std::printf("FAIL [%s] %s:%d: %s\n", g_test, __FILE__, __LINE__, #c); } \
  } while (0)
#define ASSERT_EQUAL(a, b) ASSERT_TRUE((a) == (b))

static void ReachedThroughTheVectorHeaders() {
  g_test = "ReachedThroughTheVectorHeaders";
  thrust::device_vector<int> d(1000);
  thrust::fill(d.begin(), d.end(), 3);
  ASSERT_EQUAL(thrust::reduce(d.begin(), d.end()), 3000);
  ASSERT_EQUAL(thrust::distance(d.begin(), d.end()), 1000);
  thrust::host_vector<int> h(1000);
  thrust::copy(d.begin(), d.end(), h.begin());
  ASSERT_TRUE(thrust::equal(h.begin(), h.end(), d.begin()));
  assert(h[999] == 3);  // <cassert> comes with the headers too
}

#include <thrust/allocate_unique.h>
#include <thrust/count.h>
#include <thrust/device_make_unique.h>
#include <thrust/universal_ptr.h>
#include <thrust/universal_vector.h>
#include <thrust/detail/raw_reference_cast.h>
#include <thrust/extrema.h>
#include <thrust/for_each.h>
#include <thrust/functional.h>
#include <thrust/gather.h>
#include <thrust/iterator/constant_iterator.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/iterator_adaptor.h>
#include <thrust/iterator/iterator_facade.h>
#include <thrust/iterator/permutation_iterator.h>
#include <thrust/iterator/transform_input_output_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/logical.h>
#include <thrust/memory.h>
#include <thrust/mr/allocator.h>
#include <thrust/mr/new.h>
#include <thrust/mr/polymorphic_adaptor.h>
#include <thrust/scan.h>
#include <thrust/scatter.h>
#include <thrust/sequence.h>
#include <thrust/sort.h>
#include <thrust/tuple.h>
#include <thrust/unique.h>
#include <thrust/version.h>

#include <cstdint>
#include <list>

template <typename A, typename B>
static bool same(const A& a, const B& b) {
  if (a.size() != b.size()) return false;
  for (size_t i = 0; i < a.size(); ++i)
    if (!(a[i] == b[i])) return false;
  return true;
}

// ordered by the key alone, compared for identity by both members
struct keyed {
  int key, value;
  __host__ __device__ bool operator<(const keyed& o) const { return key < o.key; }
  __host__ __device__ bool operator>(const keyed& o) const { return key > o.key; }
  bool same_as(const keyed& o) const { return key == o.key && value == o.value; }
};

template <typename T>
static void MinAndMax() {
  g_test = "MinAndMax";
  const T two(2), three(3);
  ASSERT_EQUAL(two, thrust::min THRUST_PREVENT_MACRO_SUBSTITUTION(two, three));
  ASSERT_EQUAL(two, thrust::min(three, two));
  ASSERT_EQUAL(two, thrust::min(two, three, thrust::less<T>()));
  ASSERT_EQUAL(three, thrust::min(two, three, thrust::greater<T>()));
  ASSERT_EQUAL(three, thrust::min(three, two, thrust::greater<T>()));
  ASSERT_EQUAL(three, thrust::max THRUST_PREVENT_MACRO_SUBSTITUTION(two, three));
  ASSERT_EQUAL(three, thrust::max(three, two));
  ASSERT_EQUAL(three, thrust::max(three, two, thrust::less<T>()));
  ASSERT_EQUAL(two, thrust::max(two, three, thrust::greater<T>()));
  ASSERT_EQUAL(two, thrust::max(three, two, thrust::greater<T>()));
  // of two equivalent values the first argument
  const keyed a = {2, 2}, b = {2, 3};
  ASSERT_TRUE(a.same_as(thrust::min(a, b)));
  ASSERT_TRUE(b.same_as(thrust::min(b, a)));
  ASSERT_TRUE(a.same_as(thrust::max(a, b)));
  ASSERT_TRUE(b.same_as(thrust::max(b, a)));
  ASSERT_TRUE(a.same_as(thrust::min(a, b, thrust::greater<keyed>())));
  ASSERT_TRUE(b.same_as(thrust::max(b, a, thrust::greater<keyed>())));
}

static void Distance() {
  g_test = "Distance";
  thrust::host_vector<int> h(100);
  thrust::device_vector<int> d(100);
  ASSERT_EQUAL(thrust::distance(h.begin(), h.end()), 100);
  ASSERT_EQUAL(thrust::distance(h.begin(), h.begin() + 6), 6);
  ASSERT_EQUAL(thrust::distance(d.begin(), d.end()), 100);
  ASSERT_EQUAL(thrust::distance(d.begin() + 10, d.begin() + 6), -4);
  ASSERT_EQUAL(thrust::distance(thrust::counting_iterator<int>(5), thrust::counting_iterator<int>(25)), 20);
  std::list<int> l(7);  // no subtraction: walked
  ASSERT_EQUAL(thrust::distance(l.begin(), l.end()), 7);
}

static void Version() {
  g_test = "Version";
  ASSERT_EQUAL(THRUST_VERSION, THRUST_MAJOR_VERSION * 100000 + THRUST_MINOR_VERSION * 100 + THRUST_SUBMINOR_VERSION);
  ASSERT_TRUE(THRUST_MAJOR_VERSION >= 1);
  ASSERT_TRUE(THRUST_PATCH_NUMBER >= 0);
}

static void Memory() {
  g_test = "Memory";
  const std::ptrdiff_t n = 9001;
  using namespace thrust::placeholders;
  {
    thrust::device_system_tag dev;
    typedef thrust::pointer<int, thrust::device_system_tag> pointer;
    thrust::pair<pointer, std::ptrdiff_t> got = thrust::get_temporary_buffer<int>(dev, n);
    ASSERT_EQUAL(got.second, n);
    thrust::fill_n(got.first, n, 13);
    ASSERT_TRUE(thrust::all_of(got.first, got.first + n, _1 == 13));
    thrust::return_temporary_buffer(dev, got.first, got.second);

    pointer p = pointer(static_cast<int*>(thrust::malloc(dev, sizeof(int) * n).get()));
    thrust::fill_n(p, n, 7);
    ASSERT_TRUE(thrust::all_of(p, p + n, _1 == 7));
    thrust::free(dev, p);
    pointer q = thrust::malloc<int>(dev, n);
    thrust::sequence(q, q + n);
    ASSERT_EQUAL(thrust::reduce(q, q + n, 0ll), (long long)n * (n - 1) / 2);
    thrust::free(dev, q);
  }
  {
    thrust::host_system_tag host;
    typedef thrust::pointer<int, thrust::host_system_tag> pointer;
    thrust::pair<pointer, std::ptrdiff_t> got = thrust::get_temporary_buffer<int>(host, n);
    ASSERT_EQUAL(got.second, n);
    thrust::fill_n(thrust::host, got.first, n, 13);
    ASSERT_TRUE(thrust::all_of(thrust::host, got.first, got.first + n, _1 == 13));
    thrust::return_temporary_buffer(host, got.first, got.second);
  }
}

template <typename Vector>
static void TransformInputOutputIterator() {
  g_test = "TransformInputOutputIterator";
  typedef typename Vector::value_type T;
  typedef typename Vector::iterator Iterator;
  Vector input(4), squared(4), negated(4);
  thrust::sequence(input.begin(), input.end(), 1);
  thrust::transform_input_output_iterator<thrust::negate<T>, thrust::square<T>, Iterator> it(
      squared.begin(), thrust::negate<T>(), thrust::square<T>());
  thrust::copy(input.begin(), input.end(), it);  // writes store the square
  const T gold_squared[] = {1, 4, 9, 16}, gold_negated[] = {-1, -4, -9, -16};
  ASSERT_TRUE(same(squared, thrust::host_vector<T>(gold_squared, gold_squared + 4)));
  thrust::copy_n(it, squared.size(), negated.begin());  // reads give the negation of what is stored
  ASSERT_TRUE(same(negated, thrust::host_vector<T>(gold_negated, gold_negated + 4)));

  // made by the helper, as input and output of one transform: negate(1) * 2 -> squared on the way in
  Vector out(4);
  auto from = thrust::make_transform_input_output_iterator(input.begin(), thrust::negate<T>(), thrust::square<T>());
  auto to = thrust::make_transform_input_output_iterator(out.begin(), thrust::negate<T>(), thrust::square<T>());
  using namespace thrust::placeholders;
  thrust::transform(from, from + 4, to, _1 * T(2));
  const T gold_both[] = {4, 16, 36, 64};
  ASSERT_TRUE(same(out, thrust::host_vector<T>(gold_both, gold_both + 4)));
  ASSERT_EQUAL(thrust::reduce(from, from + 4), T(-10));
}

struct clamps {
  int lo, hi;
  __host__ __device__ int operator()(int x) const { return x < lo ? lo : (hi < x ? hi : x); }
};
struct widens {
  __host__ __device__ long long operator()(int x) const { return (long long)x << 33; }
};
template <typename Vector>
static void TransformIteratorWithNamedTypes() {
  g_test = "TransformIteratorWithNamedTypes";
  Vector v(10);
  thrust::sequence(v.begin(), v.end());
  typedef typename Vector::iterator It;
  const clamps c = {2, 6};
  // Reference and Value named by the caller
  thrust::transform_iterator<clamps, It, int, int> first(v.begin(), c);
  ASSERT_EQUAL(thrust::reduce(first, first + 10), 2 + 2 + 2 + 3 + 4 + 5 + 6 + 6 + 6 + 6);
  static_assert(std::is_same<typename thrust::iterator_value<decltype(first)>::type, int>::value, "named value type");
  // only the reference named: the value type follows it
  thrust::transform_iterator<widens, It, long long> wide(v.begin(), widens());
  static_assert(std::is_same<typename thrust::iterator_value<decltype(wide)>::type, long long>::value, "from reference");
  ASSERT_EQUAL(thrust::reduce(wide, wide + 10), 45ll << 33);
  // neither: what the function returns
  auto plain = thrust::make_transform_iterator(v.begin(), widens());
  static_assert(std::is_same<typename thrust::iterator_value<decltype(plain)>::type, long long>::value, "worked out");
  ASSERT_EQUAL(thrust::reduce(plain, plain + 10), 45ll << 33);
}

// copies element i of one range to the other, through iterators it holds itself
template <typename In, typename Out>
struct copies_at {
  In in;
  Out out;
  __host__ __device__ void operator()(int i) {
    thrust::raw_reference_cast(*(out + i)) = thrust::raw_reference_cast(*(in + i));
  }
};
template <typename In, typename Out>
struct adds_at {
  In in;
  Out out;
  __host__ __device__ void operator()(int i) { out[i] += in[i]; }  // through the proxies
};
template <typename Vector, typename System>
static void IteratorsInsideFunctors() {
  g_test = "IteratorsInsideFunctors";
  typedef typename Vector::iterator It;
  Vector a(5000), b(5000, 0);
  thrust::sequence(a.begin(), a.end());
  const copies_at<It, It> f = {a.begin(), b.begin()};
  // (the counting range names its system: nothing else in the call says where to run)
  thrust::for_each(thrust::counting_iterator<int, System>(0), thrust::counting_iterator<int, System>(5000), f);
  ASSERT_TRUE(same(thrust::host_vector<int>(a), thrust::host_vector<int>(b)));
  const adds_at<It, It> g = {a.begin(), b.begin()};
  thrust::for_each(thrust::counting_iterator<int, System>(0), thrust::counting_iterator<int, System>(5000), g);
  thrust::host_vector<int> h(b);
  bool doubled = true;
  for (int i = 0; i < 5000; ++i) doubled &= h[i] == 2 * i;
  ASSERT_TRUE(doubled);
}

struct every_kth {
  long long k;
  __host__ __device__ long long operator()(long long i) const { return i * k; }
};
template <typename Vector>
static void FillThroughAStridedView() {
  g_test = "FillThroughAStridedView";
  Vector v(8);
  thrust::sequence(v.begin(), v.end(), 10, 10);  // 10 20 ... 80
  const every_kth by_two = {2};
  auto strides = thrust::make_transform_iterator(thrust::counting_iterator<long long>(0), by_two);
  auto odd = thrust::make_permutation_iterator(v.begin() + 1, strides);
  auto even = thrust::make_permutation_iterator(v.begin(), strides);
  ASSERT_EQUAL(thrust::reduce(even, even + 4), 160);
  ASSERT_EQUAL(thrust::reduce(odd, odd + 4), 200);
  thrust::fill(odd, odd + 4, 0);
  const int gold[] = {10, 0, 30, 0, 50, 0, 70, 0};
  ASSERT_TRUE(same(v, thrust::host_vector<int>(gold, gold + 8)));
  // a zip of two arrays takes a tuple
  Vector x(100, 1), y(100, 2);
  auto both = thrust::make_zip_iterator(thrust::make_tuple(x.begin(), y.begin()));
  thrust::fill(both + 10, both + 90, thrust::make_tuple(7, 9));
  ASSERT_EQUAL(thrust::reduce(x.begin(), x.end()), 20 + 80 * 7);
  ASSERT_EQUAL(thrust::reduce(y.begin(), y.end()), 40 + 80 * 9);
}

// operator() is not const: the algorithms call a copy
struct odd_counting_calls {
  int calls;
  __host__ __device__ bool operator()(int x) {
    ++calls;
    return (x & 1) != 0;
  }
};
struct by_magnitude {
  int calls;
  __host__ __device__ bool operator()(int a, int b) {
    ++calls;
    return (a < 0 ? -a : a) < (b < 0 ? -b : b);
  }
};
template <typename Vector>
static void CallablesThatAreNotConst() {
  g_test = "CallablesThatAreNotConst";
  Vector v(1001);
  thrust::sequence(v.begin(), v.end(), -500);
  odd_counting_calls odd = {0};
  ASSERT_EQUAL(thrust::count_if(v.begin(), v.end(), odd), 500);
  Vector kept(1001);
  ASSERT_EQUAL(thrust::copy_if(v.begin(), v.end(), kept.begin(), odd) - kept.begin(), 500);
  by_magnitude order = {0};
  ASSERT_EQUAL(*thrust::min_element(v.begin(), v.end(), order), 0);
  ASSERT_EQUAL(*thrust::max_element(v.begin(), v.end(), order), -500);  // of -500 and 500 the first
  thrust::sort(v.begin(), v.end(), order);
  ASSERT_EQUAL(v[0], 0);
  ASSERT_TRUE((int)v[1000] == 500 || (int)v[1000] == -500);
  ASSERT_TRUE(thrust::is_sorted(v.begin(), v.end(), order));
}

template <typename Vector>
static void UniqueOverTuples() {
  g_test = "UniqueOverTuples";
  static_assert(sizeof(thrust::tuple<float, float>) == 8, "a tuple of two floats is two floats");
  static_assert(sizeof(thrust::tuple<int>) == 4, "no room for the empty tail");
  typedef thrust::tuple<float, float> point;
  // two triangles that share an edge, as a mesh file lists them
  const point listed[] = {point(0, 0), point(1, 0), point(0, 1), point(1, 0), point(1, 1), point(0, 1)};
  Vector input(listed, listed + 6), vertices(input);
  thrust::sort(vertices.begin(), vertices.end());
  vertices.erase(thrust::unique(vertices.begin(), vertices.end()), vertices.end());
  ASSERT_EQUAL(vertices.size(), 4u);
  const point gold[] = {point(0, 0), point(0, 1), point(1, 0), point(1, 1)};
  thrust::host_vector<point> h(vertices);
  for (int i = 0; i < 4; ++i) ASSERT_TRUE(h[i] == gold[i]);
  // many points, few distinct
  const int n = 20000;
  thrust::host_vector<point> many(n);
  for (int i = 0; i < n; ++i) many[i] = point((float)((i * 7919) % 13), (float)((i * 104729) % 11));
  Vector dm(many);
  thrust::sort(dm.begin(), dm.end());
  const size_t distinct = thrust::unique(dm.begin(), dm.end()) - dm.begin();
  std::sort(many.begin(), many.end());
  const size_t gold_distinct = std::unique(many.begin(), many.end()) - many.begin();
  ASSERT_EQUAL(distinct, gold_distinct);
  thrust::host_vector<point> back(dm.begin(), dm.begin() + distinct);
  bool all = true;
  for (size_t i = 0; i < distinct; ++i) all &= back[i] == many[i];
  ASSERT_TRUE(all);
}

// counts[i] copies of values[i]: a scan gives where each run starts, a conditional scatter of the
// run numbers marks the starts, a running maximum spreads them, a gather fetches the values
template <typename Vector>
static void ExpandByCounts() {
  g_test = "ExpandByCounts";
  const int counts_in[] = {3, 5, 2, 0, 1, 3, 4, 2, 4}, values_in[] = {1, 2, 3, 4, 5, 6, 7, 8, 9};
  Vector counts(counts_in, counts_in + 9), values(values_in, values_in + 9);
  const int total = thrust::reduce(counts.begin(), counts.end());
  Vector starts(9), run_of(total, 0), output(total);
  thrust::exclusive_scan(counts.begin(), counts.end(), starts.begin());
  thrust::scatter_if(thrust::counting_iterator<int>(0), thrust::counting_iterator<int>(9), starts.begin(),
                     counts.begin(), run_of.begin());
  thrust::inclusive_scan(run_of.begin(), run_of.end(), run_of.begin(), thrust::maximum<int>());
  thrust::gather(run_of.begin(), run_of.end(), values.begin(), output.begin());
  const int gold[] = {1, 1, 1, 2, 2, 2, 2, 2, 3, 3, 5, 6, 6, 6, 7, 7, 7, 7, 8, 8, 9, 9, 9, 9};
  ASSERT_EQUAL(total, 24);
  ASSERT_TRUE(same(output, thrust::host_vector<int>(gold, gold + 24)));
}

template <typename Vector>
static void fills_and_sums(typename Vector::allocator_type alloc) {
  Vector v(alloc);
  v.resize(1000);
  thrust::sequence(v.begin(), v.end());
  ASSERT_EQUAL(thrust::reduce(v.begin(), v.end()), 499500);
  Vector w(v, alloc);
  w.push_back(500);
  ASSERT_EQUAL(thrust::reduce(w.begin(), w.end()), 500000);
}
// counts what passes through, on top of new / delete
class counting_resource final : public thrust::mr::memory_resource<void*> {
 public:
  int allocations = 0, deallocations = 0;

 protected:
  void* do_allocate(std::size_t bytes, std::size_t alignment) override {
    ++allocations;
    return below_.allocate(bytes, alignment);
  }
  void do_deallocate(void* p, std::size_t bytes, std::size_t alignment) override {
    ++deallocations;
    below_.deallocate(p, bytes, alignment);
  }

 private:
  thrust::mr::new_delete_resource below_;
};
static void AllocatorsOverChosenResources() {
  g_test = "AllocatorsOverChosenResources";
  {
    counting_resource counted;
    thrust::mr::polymorphic_adaptor_resource<void*> adaptor(&counted);
    typedef thrust::mr::polymorphic_allocator<int, void*> Alloc;
    Alloc alloc(&adaptor);
    fills_and_sums<thrust::host_vector<int, Alloc> >(alloc);
    ASSERT_TRUE(counted.allocations >= 2);
    ASSERT_EQUAL(counted.allocations, counted.deallocations);
    thrust::mr::polymorphic_adaptor_resource<void*> again(&counted);
    ASSERT_TRUE(adaptor == again);  // the same memory behind both
  }
  {
    typedef thrust::device_ptr_memory_resource<thrust::device_memory_resource> Resource;
    thrust::mr::polymorphic_adaptor_resource<thrust::device_ptr<void> > adaptor(
        thrust::mr::get_global_resource<Resource>());
    typedef thrust::mr::polymorphic_allocator<int, thrust::device_ptr<void> > Alloc;
    Alloc alloc(&adaptor);
    fills_and_sums<thrust::device_vector<int, Alloc> >(alloc);
  }
}

// Each element of the wrapped range `times` times over: only dereference() is written anew
// (the use the documentation of thrust/iterator/iterator_adaptor.h shows).
template <typename It>
class repeats : public thrust::iterator_adaptor<repeats<It>, It> {
 public:
  typedef thrust::iterator_adaptor<repeats<It>, It> super_t;
  __host__ __device__ repeats(const It& x, int times) : super_t(x), begin_(x), times_(times) {}
  friend class thrust::iterator_core_access;

 private:
  It begin_;
  int times_;
  __host__ __device__ typename super_t::reference dereference() const {
    return *(begin_ + (this->base() - begin_) / times_);
  }
};
// Every `stride`-th element of the wrapped range: movement is written anew, dereference is the
// wrapped iterator's, so the view can be written through.
template <typename It>
class strides_over : public thrust::iterator_adaptor<strides_over<It>, It> {
 public:
  typedef thrust::iterator_adaptor<strides_over<It>, It> super_t;
  typedef typename super_t::difference_type difference_type;
  __host__ __device__ strides_over(const It& x, difference_type stride) : super_t(x), stride_(stride) {}
  friend class thrust::iterator_core_access;

 private:
  difference_type stride_;
  __host__ __device__ void advance(difference_type n) { this->base_reference() += n * stride_; }
  __host__ __device__ void increment() { this->base_reference() += stride_; }
  __host__ __device__ void decrement() { this->base_reference() -= stride_; }
  __host__ __device__ difference_type distance_to(const strides_over& o) const {
    return (o.base() - this->base()) / stride_;
  }
};
// a * i + b for i = 0, 1, ...: nothing wrapped, every member written here
template <typename System>
class affine : public thrust::iterator_facade<affine<System>, long long, System, thrust::random_access_traversal_tag,
                                              long long, std::ptrdiff_t> {
 public:
  __host__ __device__ affine(long long a, long long b, std::ptrdiff_t i = 0) : a_(a), b_(b), i_(i) {}
  friend class thrust::iterator_core_access;

 private:
  long long a_, b_;
  std::ptrdiff_t i_;
  __host__ __device__ long long dereference() const { return a_ * i_ + b_; }
  __host__ __device__ bool equal(const affine& o) const { return i_ == o.i_; }
  __host__ __device__ void increment() { ++i_; }
  __host__ __device__ void decrement() { --i_; }
  __host__ __device__ void advance(std::ptrdiff_t n) { i_ += n; }
  __host__ __device__ std::ptrdiff_t distance_to(const affine& o) const { return o.i_ - i_; }
};

template <typename Vector, typename System>
static void IteratorsOfTheCallersOwn() {
  g_test = "IteratorsOfTheCallersOwn";
  typedef typename Vector::iterator It;
  static_assert(std::is_same<typename thrust::iterator_system<repeats<It> >::type, System>::value, "the wrapped iterator's system");
  static_assert(std::is_same<typename thrust::iterator_value<repeats<It> >::type, int>::value, "the wrapped iterator's value");
  const int few[] = {10, 20, 30, 40};
  Vector v(few, few + 4);
  repeats<It> first(v.begin(), 3), last(v.end(), 3);
  ASSERT_EQUAL(first[0], 10);
  ASSERT_EQUAL(first[2], 10);
  ASSERT_EQUAL(first[3], 20);
  ASSERT_EQUAL(*(first + 11), 40);
  ASSERT_EQUAL((first + 12) - first, 12);
  Vector out(12);
  thrust::copy(first, first + 12, out.begin());
  const int gold[] = {10, 10, 10, 20, 20, 20, 30, 30, 30, 40, 40, 40};
  ASSERT_TRUE(same(out, thrust::host_vector<int>(gold, gold + 12)));
  ASSERT_EQUAL(thrust::reduce(first, first + 12), 300);
  (void)last;
  // a long one, against the closed form
  Vector big(5000);
  thrust::sequence(big.begin(), big.end());
  repeats<It> rb(big.begin(), 7);
  ASSERT_EQUAL(thrust::reduce(rb, rb + 35000, 0ll), 7ll * 4999 * 5000 / 2);
  using namespace thrust::placeholders;
  Vector twice(35000);
  thrust::transform(rb, rb + 35000, twice.begin(), _1 * 2);
  ASSERT_EQUAL((int)twice[34999], 9998);
  ASSERT_EQUAL((int)twice[7], 2);

  // written through: every third element
  Vector w(30, 1);
  strides_over<It> s(w.begin(), 3);
  ASSERT_EQUAL((s + 10) - s, 10);
  thrust::fill(s, s + 10, 5);
  ASSERT_EQUAL(thrust::reduce(w.begin(), w.end()), 20 + 50);
  ASSERT_EQUAL((int)w[0], 5);
  ASSERT_EQUAL((int)w[1], 1);
  ASSERT_EQUAL((int)w[27], 5);
  thrust::transform(s, s + 10, thrust::counting_iterator<int>(0), s, _1 + _2);  // in place through the view
  ASSERT_EQUAL((int)w[27], 14);
  ASSERT_EQUAL((int)w[28], 1);
  ASSERT_EQUAL(thrust::reduce(s, s + 10), 50 + 45);

  // nothing wrapped
  affine<System> a(3, 1);
  ASSERT_EQUAL(*a, 1);
  ASSERT_EQUAL(a[4], 13);
  ASSERT_EQUAL(thrust::reduce(a, a + 100000), 3ll * 99999 * 100000 / 2 + 100000);
  thrust::host_vector<long long> got(5);
  thrust::copy(a + 2, a + 7, got.begin());
  ASSERT_EQUAL(got[0], 7);
  ASSERT_EQUAL(got[4], 19);
  ASSERT_EQUAL(thrust::count_if(a, a + 1000, _1 % 2 == 0), 500);
}

template <typename T>
struct holds {
  T held;
  holds(T x) : held(x) {}
  __host__ __device__ T getter() const { return held; }
};
template <typename T>
static void OwnedThroughUniquePtr() {
  g_test = "OwnedThroughUniquePtr";
  {  // storage the host addresses too: read through the pointer (testing/universal_memory.cu:35-66)
    auto raw = thrust::allocate_unique<T>(thrust::universal_allocator<T>(), 42);
    auto obj = thrust::allocate_unique<holds<T> >(thrust::universal_allocator<holds<T> >(), 42);
    static_assert(std::is_same<decltype(raw.get()), thrust::universal_ptr<T> >::value, "the allocator's pointer");
    static_assert(std::is_same<decltype(obj.get()), thrust::universal_ptr<holds<T> > >::value, "the allocator's pointer");
    // (through get(): std::unique_ptr's own operator* wants a plain T&, and what a device_ptr
    // yields on the host is a proxy)
    ASSERT_EQUAL((T)*raw.get(), T(42));
    ASSERT_EQUAL((T)raw.get()[0], T(42));
    ASSERT_EQUAL(obj->getter(), T(42));
    ASSERT_EQUAL(obj.get()->getter(), T(42));
    auto array = thrust::allocate_unique_n<T>(thrust::universal_allocator<T>(), 6, 42);
    static_assert(std::is_same<decltype(array.get()), thrust::universal_ptr<T> >::value, "the allocator's pointer");
    ASSERT_EQUAL(thrust::reduce(array.get(), array.get() + 6), T(6 * 42));
    ASSERT_EQUAL(array.get_deleter().size(), 6u);
    for (int i = 0; i < 6; ++i) array.get()[i] = T(i);  // written by the host ...
    ASSERT_EQUAL(thrust::reduce(array.get(), array.get() + 6), T(15));  // ... summed by the device
  }
  {  // device memory
    auto one = thrust::device_make_unique<T>(T(7));
    static_assert(std::is_same<decltype(one.get()), thrust::device_ptr<T> >::value, "device_allocator's pointer");
    ASSERT_EQUAL((T)*one.get(), T(7));
    auto zero = thrust::device_make_unique<T>();
    ASSERT_EQUAL((T)*zero.get(), T());
    auto many = thrust::allocate_unique_n<T>(thrust::device_allocator<T>(), 1000, 3);
    ASSERT_EQUAL(thrust::reduce(many.get(), many.get() + 1000), T(3000));
    auto blank = thrust::uninitialized_allocate_unique_n<T>(thrust::device_allocator<T>(), 1000);
    thrust::copy(many.get(), many.get() + 1000, blank.get());
    ASSERT_TRUE(thrust::equal(many.get(), many.get() + 1000, blank.get()));
    one.reset();  // gives the storage back now
    ASSERT_TRUE(!one);
  }
  {  // the host's allocator: constructed in place, destroyed on release
    static int alive;
    alive = 0;
    struct counted {
      counted(int) { ++alive; }
      counted(const counted&) { ++alive; }
      ~counted() { --alive; }
    };
    {
      auto one = thrust::allocate_unique<counted>(std::allocator<counted>(), 1);
      ASSERT_EQUAL(alive, 1);
      auto five = thrust::allocate_unique_n<counted>(std::allocator<counted>(), 5, 1);
      ASSERT_EQUAL(alive, 6);
    }
    ASSERT_EQUAL(alive, 0);
  }
}

int main() {
  ReachedThroughTheVectorHeaders();
  MinAndMax<int>();
  MinAndMax<float>();
  MinAndMax<long long>();
  MinAndMax<unsigned char>();
  Distance();
  Version();
  Memory();
  TransformInputOutputIterator<thrust::host_vector<int> >();
  TransformInputOutputIterator<thrust::device_vector<int> >();
  TransformInputOutputIterator<thrust::device_vector<float> >();
  TransformIteratorWithNamedTypes<thrust::host_vector<int> >();
  TransformIteratorWithNamedTypes<thrust::device_vector<int> >();
  IteratorsInsideFunctors<thrust::host_vector<int>, thrust::host_system_tag>();
  IteratorsInsideFunctors<thrust::device_vector<int>, thrust::device_system_tag>();
  FillThroughAStridedView<thrust::host_vector<int> >();
  FillThroughAStridedView<thrust::device_vector<int> >();
  CallablesThatAreNotConst<thrust::host_vector<int> >();
  CallablesThatAreNotConst<thrust::device_vector<int> >();
  UniqueOverTuples<thrust::host_vector<thrust::tuple<float, float> > >();
  UniqueOverTuples<thrust::device_vector<thrust::tuple<float, float> > >();
  ExpandByCounts<thrust::host_vector<int> >();
  ExpandByCounts<thrust::device_vector<int> >();
  AllocatorsOverChosenResources();
  IteratorsOfTheCallersOwn<thrust::host_vector<int>, thrust::host_system_tag>();
  IteratorsOfTheCallersOwn<thrust::device_vector<int>, thrust::device_system_tag>();
  OwnedThroughUniquePtr<int>();
  OwnedThroughUniquePtr<double>();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
