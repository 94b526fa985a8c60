// Front-end test compiled with the plain host compiler: the containers and pointer types of the
// API as the reference's own unit tests exercise them (testing/vector.cu:12-760,
// vector_insert.cu:5-300, vector_manipulation.cu:5-110, device_ptr.cu:5-125,
// device_reference.cu:5-215).  Every case runs for host_vector and for device_vector over
// several element types; literal expectations are the reference's, random cases compare the
// device container with std::vector.
#include <thrust/device_ptr.h>
#include <thrust/device_reference.h>
#include <thrust/device_vector.h>
#include <thrust/host_vector.h>
#include <thrust/sequence.h>

#include <cstdint>
#include <cstdio>
#include <list>
#include <vector>

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
static thrust::host_vector<T> random_samples(size_t n, uint64_t seed) {
  thrust::host_vector<T> h(n);
  for (size_t i = 0; i < n; ++i) h[i] = (T)(mix(seed * 1000003ull + i) % 1000);
  return h;
}

template <class Vector>
static void VectorBasics() {
  typedef typename Vector::value_type T;
  g_test = "VectorZeroSize";
  {
    Vector v;
    ASSERT_EQUAL(v.size(), 0lu);
    ASSERT_EQUAL((v.begin() == v.end()), true);
  }
  g_test = "VectorFrontBack";
  {
    Vector v(3);
    v[0] = 0; v[1] = 1; v[2] = 2;
    ASSERT_EQUAL(v.front(), T(0));
    ASSERT_EQUAL(v.back(), T(2));
  }
  g_test = "VectorData";
  {
    typedef typename Vector::pointer PointerT;
    typedef typename Vector::const_pointer PointerConstT;
    Vector v(3);
    v[0] = 0; v[1] = 1; v[2] = 2;
    ASSERT_EQUAL(T(0), *v.data());
    ASSERT_EQUAL(T(1), *(v.data() + 1));
    ASSERT_EQUAL(T(2), *(v.data() + 2));
    ASSERT_EQUAL(PointerT(&v.front()), v.data());
    ASSERT_EQUAL(PointerT(&*v.begin()), v.data());
    ASSERT_EQUAL(PointerT(&v[0]), v.data());
    const Vector& c_v = v;
    ASSERT_EQUAL(T(0), *c_v.data());
    ASSERT_EQUAL(T(1), *(c_v.data() + 1));
    ASSERT_EQUAL(T(2), *(c_v.data() + 2));
    ASSERT_EQUAL(PointerConstT(&c_v.front()), c_v.data());
    ASSERT_EQUAL(PointerConstT(&*c_v.begin()), c_v.data());
    ASSERT_EQUAL(PointerConstT(&c_v[0]), c_v.data());
  }
  g_test = "VectorElementAssignment";
  {
    Vector v(3);
    v[0] = 0; v[1] = 1; v[2] = 2;
    ASSERT_EQUAL(v[0], T(0)); ASSERT_EQUAL(v[1], T(1)); ASSERT_EQUAL(v[2], T(2));
    v[0] = 10; v[1] = 11; v[2] = 12;
    ASSERT_EQUAL(v[0], T(10)); ASSERT_EQUAL(v[1], T(11)); ASSERT_EQUAL(v[2], T(12));
    Vector w(3);
    w[0] = v[0];
    w[1] = v[1];
    w[2] = v[2];
    ASSERT_EQUAL(v, w);
  }
  g_test = "VectorFromSTLVector / AssignFromSTLVector / FillAssign";
  {
    std::vector<T> stl_vector(3);
    stl_vector[0] = 0; stl_vector[1] = 1; stl_vector[2] = 2;
    Vector v(stl_vector);
    ASSERT_EQUAL(v.size(), 3lu);
    ASSERT_EQUAL(v[0], T(0)); ASSERT_EQUAL(v[1], T(1)); ASSERT_EQUAL(v[2], T(2));
    v = stl_vector;
    ASSERT_EQUAL(v.size(), 3lu);
    ASSERT_EQUAL(v[0], T(0)); ASSERT_EQUAL(v[1], T(1)); ASSERT_EQUAL(v[2], T(2));
    Vector a;
    a.assign(stl_vector.begin(), stl_vector.end());
    ASSERT_EQUAL(a.size(), 3lu);
    ASSERT_EQUAL(a[0], T(0)); ASSERT_EQUAL(a[1], T(1)); ASSERT_EQUAL(a[2], T(2));
    Vector f;
    f.assign(3, 13);
    ASSERT_EQUAL(f.size(), 3lu);
    ASSERT_EQUAL(f[0], T(13)); ASSERT_EQUAL(f[1], T(13)); ASSERT_EQUAL(f[2], T(13));
  }
  g_test = "VectorFromBiDirectionalIterator / AssignFromBiDirectionalIterator";
  {
    std::list<T> stl_list;
    stl_list.push_back(0); stl_list.push_back(1); stl_list.push_back(2);
    Vector v(stl_list.begin(), stl_list.end());
    ASSERT_EQUAL(v.size(), 3lu);
    ASSERT_EQUAL(v[0], T(0)); ASSERT_EQUAL(v[1], T(1)); ASSERT_EQUAL(v[2], T(2));
    Vector a;
    a.assign(stl_list.begin(), stl_list.end());
    ASSERT_EQUAL(a.size(), 3lu);
    ASSERT_EQUAL(a[0], T(0)); ASSERT_EQUAL(a[1], T(1)); ASSERT_EQUAL(a[2], T(2));
  }
  g_test = "VectorAssignFromHostVector / ToAndFromHostVector";
  {
    thrust::host_vector<T> h(3);
    h[0] = 0; h[1] = 1; h[2] = 2;
    Vector a;
    a.assign(h.begin(), h.end());
    ASSERT_EQUAL(a, h);
    Vector v(h);
    ASSERT_EQUAL(v, h);
    Vector& self = v;
    v = self;
    ASSERT_EQUAL(v, h);
    v[0] = 10; v[1] = 11; v[2] = 12;
    ASSERT_EQUAL(h[0], T(0)); ASSERT_EQUAL(v[0], T(10));
    ASSERT_EQUAL(h[1], T(1)); ASSERT_EQUAL(v[1], T(11));
    ASSERT_EQUAL(h[2], T(2)); ASSERT_EQUAL(v[2], T(12));
    h = v;
    ASSERT_EQUAL(v, h);
    h[1] = 11;
    v = h;
    ASSERT_EQUAL(v, h);
  }
  g_test = "VectorAssignFromDeviceVector / ToAndFromDeviceVector";
  {
    thrust::device_vector<T> d(3);
    d[0] = 0; d[1] = 1; d[2] = 2;
    Vector a;
    a.assign(d.begin(), d.end());
    ASSERT_EQUAL(a, d);
    Vector v(d);
    ASSERT_EQUAL(v, d);
    v[0] = 10; v[1] = 11; v[2] = 12;
    ASSERT_EQUAL(d[0], T(0)); ASSERT_EQUAL(v[0], T(10));
    ASSERT_EQUAL(d[1], T(1)); ASSERT_EQUAL(v[1], T(11));
    ASSERT_EQUAL(d[2], T(2)); ASSERT_EQUAL(v[2], T(12));
    d = v;
    ASSERT_EQUAL(v, d);
    d[1] = 11;
    v = d;
    ASSERT_EQUAL(v, d);
  }
  g_test = "VectorWithInitialValue";
  {
    const T init = 17;
    Vector v(3, init);
    ASSERT_EQUAL(v.size(), 3lu);
    ASSERT_EQUAL(v[0], init); ASSERT_EQUAL(v[1], init); ASSERT_EQUAL(v[2], init);
  }
  g_test = "VectorSwap";
  {
    Vector v(3);
    v[0] = 0; v[1] = 1; v[2] = 2;
    Vector u(3);
    u[0] = 10; u[1] = 11; u[2] = 12;
    v.swap(u);
    ASSERT_EQUAL(v[0], T(10)); ASSERT_EQUAL(u[0], T(0));
    ASSERT_EQUAL(v[1], T(11)); ASSERT_EQUAL(u[1], T(1));
    ASSERT_EQUAL(v[2], T(12)); ASSERT_EQUAL(u[2], T(2));
  }
  g_test = "VectorErasePosition";
  {
    Vector v(5);
    v[0] = 0; v[1] = 1; v[2] = 2; v[3] = 3; v[4] = 4;
    v.erase(v.begin() + 2);
    ASSERT_EQUAL(v.size(), 4lu);
    ASSERT_EQUAL(v[0], T(0)); ASSERT_EQUAL(v[1], T(1)); ASSERT_EQUAL(v[2], T(3)); ASSERT_EQUAL(v[3], T(4));
    v.erase(v.begin() + 0);
    ASSERT_EQUAL(v.size(), 3lu);
    ASSERT_EQUAL(v[0], T(1)); ASSERT_EQUAL(v[1], T(3)); ASSERT_EQUAL(v[2], T(4));
    v.erase(v.begin() + 2);
    ASSERT_EQUAL(v.size(), 2lu);
    ASSERT_EQUAL(v[0], T(1)); ASSERT_EQUAL(v[1], T(3));
    v.erase(v.begin() + 1);
    ASSERT_EQUAL(v.size(), 1lu);
    ASSERT_EQUAL(v[0], T(1));
    v.erase(v.begin() + 0);
    ASSERT_EQUAL(v.size(), 0lu);
  }
  g_test = "VectorEraseRange";
  {
    Vector v(6);
    v[0] = 0; v[1] = 1; v[2] = 2; v[3] = 3; v[4] = 4; v[5] = 5;
    v.erase(v.begin() + 1, v.begin() + 3);
    ASSERT_EQUAL(v.size(), 4lu);
    ASSERT_EQUAL(v[0], T(0)); ASSERT_EQUAL(v[1], T(3)); ASSERT_EQUAL(v[2], T(4)); ASSERT_EQUAL(v[3], T(5));
    v.erase(v.begin() + 2, v.end());
    ASSERT_EQUAL(v.size(), 2lu);
    ASSERT_EQUAL(v[0], T(0)); ASSERT_EQUAL(v[1], T(3));
    v.erase(v.begin() + 0, v.begin() + 1);
    ASSERT_EQUAL(v.size(), 1lu);
    ASSERT_EQUAL(v[0], T(3));
    v.erase(v.begin(), v.end());
    ASSERT_EQUAL(v.size(), 0lu);
  }
  g_test = "VectorResizing / Reserving / ShrinkToFit";
  {
    Vector v;
    v.resize(3);
    ASSERT_EQUAL(v.size(), 3lu);
    v[0] = 0; v[1] = 1; v[2] = 2;
    v.resize(5);
    ASSERT_EQUAL(v.size(), 5lu);
    ASSERT_EQUAL(v[0], T(0)); ASSERT_EQUAL(v[1], T(1)); ASSERT_EQUAL(v[2], T(2));
    v[3] = 3; v[4] = 4;
    v.resize(4);
    ASSERT_EQUAL(v.size(), 4lu);
    ASSERT_EQUAL(v[0], T(0)); ASSERT_EQUAL(v[1], T(1)); ASSERT_EQUAL(v[2], T(2)); ASSERT_EQUAL(v[3], T(3));
    v.resize(0);
    ASSERT_EQUAL(v.size(), 0lu);
    Vector r;
    r.reserve(3);
    ASSERT_TRUE(r.capacity() >= 3lu);
    const size_t old_capacity = r.capacity();
    r.reserve(0);
    ASSERT_EQUAL(r.capacity(), old_capacity);
    Vector s;
    s.reserve(200);
    ASSERT_TRUE(s.capacity() >= 200lu);
    s.push_back(1); s.push_back(2); s.push_back(3);
    s.shrink_to_fit();
    ASSERT_EQUAL(T(1), s[0]); ASSERT_EQUAL(T(2), s[1]); ASSERT_EQUAL(T(3), s[2]);
    ASSERT_EQUAL(3lu, s.size());
    ASSERT_EQUAL(3lu, s.capacity());
  }
  g_test = "VectorReversed";
  {
    Vector v(3);
    v[0] = 0; v[1] = 1; v[2] = 2;
    ASSERT_EQUAL(3, v.rend() - v.rbegin());
    ASSERT_EQUAL(3, static_cast<const Vector&>(v).rend() - static_cast<const Vector&>(v).rbegin());
    ASSERT_EQUAL(3, v.crend() - v.crbegin());
    ASSERT_EQUAL(T(2), *v.rbegin());
    ASSERT_EQUAL(T(2), *static_cast<const Vector&>(v).rbegin());
    ASSERT_EQUAL(T(2), *v.crbegin());
    ASSERT_EQUAL(T(1), *(v.rbegin() + 1));
    ASSERT_EQUAL(T(0), *(v.rbegin() + 2));
    ASSERT_EQUAL(T(0), *(v.rend() - 1));
    ASSERT_EQUAL(T(1), *(v.rend() - 2));
  }
}

template <class Vector>
static void VectorInsertSimple() {
  typedef typename Vector::value_type T;
  g_test = "VectorRangeInsertSimple";
  Vector v1(5);
  thrust::sequence(v1.begin(), v1.end());
  {
    // fits inside capacity, more inserted than displaced
    Vector v2(3);
    v2.reserve(10);
    thrust::sequence(v2.begin(), v2.end());
    ASSERT_TRUE(v2.capacity() >= v2.size() + v1.size());
    v2.insert(v2.begin() + 1, v1.begin(), v1.end());
    const T expect[8] = {0, 0, 1, 2, 3, 4, 1, 2};
    for (int i = 0; i < 8; ++i) ASSERT_EQUAL(T(expect[i]), v2[i]);
    ASSERT_EQUAL(8lu, v2.size());
    ASSERT_EQUAL(10lu, v2.capacity());
  }
  {
    // as many inserted as displaced
    Vector v3(5);
    v3.reserve(10);
    thrust::sequence(v3.begin(), v3.end());
    v3.insert(v3.begin(), v1.begin(), v1.end());
    const T expect[10] = {0, 1, 2, 3, 4, 0, 1, 2, 3, 4};
    for (int i = 0; i < 10; ++i) ASSERT_EQUAL(T(expect[i]), v3[i]);
    ASSERT_EQUAL(10lu, v3.size());
    ASSERT_EQUAL(10lu, v3.capacity());
  }
  {
    // fewer inserted than displaced
    Vector v4(5);
    v4.reserve(10);
    thrust::sequence(v4.begin(), v4.end());
    v4.insert(v4.begin() + 1, v1.begin(), v1.begin() + 3);
    const T expect[8] = {0, 0, 1, 2, 1, 2, 3, 4};
    for (int i = 0; i < 8; ++i) ASSERT_EQUAL(T(expect[i]), v4[i]);
    ASSERT_EQUAL(8lu, v4.size());
    ASSERT_EQUAL(10lu, v4.capacity());
  }
  {
    // does not fit inside capacity
    Vector v5(5);
    thrust::sequence(v5.begin(), v5.end());
    ASSERT_TRUE(v5.capacity() < v5.size() + v1.size());
    v5.insert(v5.begin() + 1, v1.begin(), v1.end());
    const T expect[10] = {0, 0, 1, 2, 3, 4, 1, 2, 3, 4};
    for (int i = 0; i < 10; ++i) ASSERT_EQUAL(T(expect[i]), v5[i]);
    ASSERT_EQUAL(10lu, v5.size());
  }
  g_test = "VectorFillInsertSimple";
  {
    Vector f1(3);
    f1.reserve(10);
    thrust::sequence(f1.begin(), f1.end());
    f1.insert(f1.begin() + 1, 5, 13);
    const T expect[8] = {0, 13, 13, 13, 13, 13, 1, 2};
    for (int i = 0; i < 8; ++i) ASSERT_EQUAL(T(expect[i]), f1[i]);
    ASSERT_EQUAL(8lu, f1.size());
    ASSERT_EQUAL(10lu, f1.capacity());
  }
  {
    Vector f2(5);
    f2.reserve(10);
    thrust::sequence(f2.begin(), f2.end());
    f2.insert(f2.begin(), 5, 13);
    const T expect[10] = {13, 13, 13, 13, 13, 0, 1, 2, 3, 4};
    for (int i = 0; i < 10; ++i) ASSERT_EQUAL(T(expect[i]), f2[i]);
    ASSERT_EQUAL(10lu, f2.size());
    ASSERT_EQUAL(10lu, f2.capacity());
  }
  {
    Vector f3(5);
    f3.reserve(10);
    thrust::sequence(f3.begin(), f3.end());
    f3.insert(f3.begin() + 1, 3, 13);
    const T expect[8] = {0, 13, 13, 13, 1, 2, 3, 4};
    for (int i = 0; i < 8; ++i) ASSERT_EQUAL(T(expect[i]), f3[i]);
    ASSERT_EQUAL(8lu, f3.size());
    ASSERT_EQUAL(10lu, f3.capacity());
  }
  {
    Vector f4(5);
    thrust::sequence(f4.begin(), f4.end());
    ASSERT_TRUE(f4.capacity() < f4.size() + 5);
    f4.insert(f4.begin() + 1, 5, 13);
    const T expect[10] = {0, 13, 13, 13, 13, 13, 1, 2, 3, 4};
    for (int i = 0; i < 10; ++i) ASSERT_EQUAL(T(expect[i]), f4[i]);
    ASSERT_EQUAL(10lu, f4.size());
  }
  g_test = "VectorInsert (single element)";
  {
    Vector s(3);
    thrust::sequence(s.begin(), s.end());
    typename Vector::iterator at = s.insert(s.begin() + 1, T(9));
    ASSERT_TRUE(at == s.begin() + 1);
    const T expect[4] = {0, 9, 1, 2};
    for (int i = 0; i < 4; ++i) ASSERT_EQUAL(T(expect[i]), s[i]);
  }
}

template <typename T>
static void VectorInsertRandom(uint64_t seed) {
  for (size_t n : {(size_t)0, (size_t)1, (size_t)2, (size_t)63, (size_t)1000, (size_t)65539}) {
    g_test = "VectorRangeInsert";
    thrust::host_vector<T> h_src = random_samples<T>(n + 3, seed + n);
    thrust::host_vector<T> h_dst = random_samples<T>(n, seed + 17 + n);
    thrust::device_vector<T> d_src = h_src;
    thrust::device_vector<T> d_dst = h_dst;
    size_t begin = n > 0 ? (size_t)h_src[n] % n : 0;
    size_t end = n > 0 ? (size_t)h_src[n + 1] % n : 0;
    if (end < begin) std::swap(begin, end);
    const size_t position = n > 0 ? (size_t)h_src[n + 2] % n : 0;
    std::vector<T> expect(h_dst.begin(), h_dst.end());
    expect.insert(expect.begin() + position, h_src.begin() + begin, h_src.begin() + end);
    h_dst.insert(h_dst.begin() + position, h_src.begin() + begin, h_src.begin() + end);
    d_dst.insert(d_dst.begin() + position, d_src.begin() + begin, d_src.begin() + end);
    ASSERT_TRUE(h_dst == expect);
    ASSERT_TRUE(d_dst == expect);
    ASSERT_EQUAL(h_dst, d_dst);
    g_test = "VectorFillInsert";
    thrust::host_vector<T> h_fill = random_samples<T>(n + 2, seed + 33 + n);
    thrust::device_vector<T> d_fill = h_fill;
    const size_t where = n > 0 ? (size_t)h_fill[n] % n : 0;
    const size_t how_many = n > 0 ? (size_t)h_fill[n] % n : 13;
    std::vector<T> expect_fill(h_fill.begin(), h_fill.end());
    expect_fill.insert(expect_fill.begin() + where, how_many, T(13));
    h_fill.insert(h_fill.begin() + where, how_many, T(13));
    d_fill.insert(d_fill.begin() + where, how_many, T(13));
    ASSERT_TRUE(h_fill == expect_fill);
    ASSERT_TRUE(d_fill == expect_fill);
  }
}

template <class Vector>
static void VectorManipulation(size_t n, uint64_t seed) {
  typedef typename Vector::iterator Iterator;
  typedef typename Vector::value_type T;
  g_test = "VectorManipulation";
  thrust::host_vector<T> src = random_samples<T>(n, seed);
  ASSERT_EQUAL(src.size(), n);
  Vector test0(n);
  Vector test1(n, T(3));
  ASSERT_EQUAL(test0.size(), n);
  ASSERT_EQUAL(test1.size(), n);
  ASSERT_EQUAL((test1 == std::vector<T>(n, T(3))), true);
  std::vector<T> stl_vector(src.begin(), src.end());
  Vector cpy0 = src;
  Vector cpy1(stl_vector);
  Vector cpy2(stl_vector.begin(), stl_vector.end());
  ASSERT_EQUAL(cpy0, src);
  ASSERT_EQUAL(cpy1, src);
  ASSERT_EQUAL(cpy2, src);
  Vector vec1(src);
  vec1.resize(n + 3);
  ASSERT_EQUAL(vec1.size(), n + 3);
  vec1.resize(n);
  ASSERT_EQUAL(vec1.size(), n);
  ASSERT_EQUAL(vec1, src);
  vec1.resize(n + 20, T(11));
  Vector tail(vec1.begin() + n, vec1.end());
  ASSERT_EQUAL((tail == std::vector<T>(20, T(11))), true);
  // shrinking a vector does not invalidate iterators
  Iterator first = vec1.begin();
  vec1.resize(10);
  ASSERT_TRUE(first == vec1.begin());
  vec1.resize(0);
  ASSERT_EQUAL(vec1.size(), 0lu);
  ASSERT_EQUAL(vec1.empty(), true);
  vec1.resize(10);
  ASSERT_EQUAL(vec1.size(), 10lu);
  vec1.clear();
  ASSERT_EQUAL(vec1.size(), 0lu);
  vec1.resize(5);
  ASSERT_EQUAL(vec1.size(), 5lu);
  Vector vec2;
  for (size_t i = 0; i < 10; ++i) {
    ASSERT_EQUAL(vec2.size(), i);
    vec2.push_back(T(i));
    ASSERT_EQUAL(vec2.size(), i + 1);
    for (size_t j = 0; j <= i; j++) ASSERT_EQUAL(vec2[j], T(j));
    ASSERT_EQUAL(vec2.back(), T(i));
  }
  for (size_t i = 10; i > 0; --i) {
    ASSERT_EQUAL(vec2.size(), i);
    ASSERT_EQUAL(vec2.back(), T(i - 1));
    vec2.pop_back();
    ASSERT_EQUAL(vec2.size(), i - 1);
    for (size_t j = 0; j + 1 < i; j++) ASSERT_EQUAL(vec2[j], T(j));
  }
}

static void TestVectorBool() {
  g_test = "VectorBool";
  thrust::host_vector<bool> h(3);
  thrust::device_vector<bool> d(3);
  h[0] = true; h[1] = false; h[2] = true;
  d[0] = true; d[1] = false; d[2] = true;
  ASSERT_EQUAL(h[0], true); ASSERT_EQUAL(h[1], false); ASSERT_EQUAL(h[2], true);
  ASSERT_EQUAL(d[0], true); ASSERT_EQUAL(d[1], false); ASSERT_EQUAL(d[2], true);
  ASSERT_EQUAL(h, d);
}

static void TestVectorEqualityAndInequality() {
  g_test = "VectorEquality / Inequality";
  thrust::host_vector<int> h_a(3), h_b(3), h_c(3);
  h_a[0] = 0; h_a[1] = 1; h_a[2] = 2;
  h_b[0] = 0; h_b[1] = 1; h_b[2] = 3;
  thrust::device_vector<int> d_a = h_a, d_b = h_b, d_c = h_c;
  std::vector<int> s_a(h_a.begin(), h_a.end()), s_b(h_b.begin(), h_b.end()), s_c(h_c.begin(), h_c.end());
  // every pairing of the three container kinds, equal and unequal contents
#define CHECK_SAME(x, y) do { ASSERT_EQUAL((x == y), true); ASSERT_EQUAL((x != y), false); } while (0)
#define CHECK_DIFFERENT(x, y) do { ASSERT_EQUAL((x == y), false); ASSERT_EQUAL((x != y), true); } while (0)
  CHECK_SAME(h_a, h_a); CHECK_SAME(h_a, d_a); CHECK_SAME(d_a, h_a); CHECK_SAME(d_a, d_a);
  CHECK_SAME(h_b, h_b); CHECK_SAME(h_b, d_b); CHECK_SAME(d_b, h_b); CHECK_SAME(d_b, d_b);
  CHECK_SAME(h_c, h_c); CHECK_SAME(h_c, d_c); CHECK_SAME(d_c, h_c); CHECK_SAME(d_c, d_c);
  CHECK_SAME(s_a, d_a); CHECK_SAME(d_a, s_a); CHECK_SAME(s_b, d_b); CHECK_SAME(d_b, s_b);
  CHECK_SAME(s_a, h_a); CHECK_SAME(h_a, s_a); CHECK_SAME(s_c, h_c); CHECK_SAME(h_c, s_c);
  CHECK_DIFFERENT(h_a, h_b); CHECK_DIFFERENT(h_a, d_b); CHECK_DIFFERENT(d_a, h_b); CHECK_DIFFERENT(d_a, d_b);
  CHECK_DIFFERENT(h_b, h_a); CHECK_DIFFERENT(h_b, d_a); CHECK_DIFFERENT(d_b, h_a); CHECK_DIFFERENT(d_b, d_a);
  CHECK_DIFFERENT(h_a, h_c); CHECK_DIFFERENT(h_a, d_c); CHECK_DIFFERENT(d_a, h_c); CHECK_DIFFERENT(d_a, d_c);
  CHECK_DIFFERENT(h_b, h_c); CHECK_DIFFERENT(h_b, d_c); CHECK_DIFFERENT(d_b, h_c); CHECK_DIFFERENT(d_b, d_c);
  CHECK_DIFFERENT(s_a, d_b); CHECK_DIFFERENT(d_a, s_b); CHECK_DIFFERENT(s_b, d_a); CHECK_DIFFERENT(d_b, s_a);
  CHECK_DIFFERENT(s_a, d_c); CHECK_DIFFERENT(d_a, s_c); CHECK_DIFFERENT(s_c, d_b); CHECK_DIFFERENT(d_c, s_b);
  CHECK_DIFFERENT(s_a, h_b); CHECK_DIFFERENT(h_a, s_b); CHECK_DIFFERENT(s_c, h_b); CHECK_DIFFERENT(h_c, s_b);
  // different sizes
  thrust::device_vector<int> d_short(2);
  d_short[0] = 0; d_short[1] = 1;
  CHECK_DIFFERENT(d_short, d_a); CHECK_DIFFERENT(h_a, d_short); CHECK_DIFFERENT(d_short, s_a);
#undef CHECK_SAME
#undef CHECK_DIFFERENT
  g_test = "VectorUninitialisedCopy";
  thrust::device_vector<int> v;
  std::vector<int> std_vector;
  v = std_vector;
  ASSERT_EQUAL(v.size(), static_cast<size_t>(0));
}

template <int N>
struct LargeStruct {
  int data[N];
  bool operator==(const LargeStruct& ls) const {
    for (int i = 0; i < N; i++)
      if (data[i] != ls.data[i]) return false;
    return true;
  }
};

static void TestVectorContainingLargeType() {
  g_test = "VectorContainingLargeType";
  const static int N = 100;
  typedef LargeStruct<N> T;
  thrust::device_vector<T> dv1;
  thrust::host_vector<T> hv1;
  ASSERT_TRUE(dv1 == hv1);
  thrust::device_vector<T> dv2(20);
  thrust::host_vector<T> hv2(20);
  ASSERT_TRUE(dv2 == hv2);
  T ls;
  for (int i = 0; i < N; i++) ls.data[i] = i;
  thrust::device_vector<T> dv3(20, ls);
  thrust::host_vector<T> hv3(20, ls);
  ASSERT_TRUE(dv3 == hv3);
  ls.data[0] = -13;
  dv3[2] = ls;
  hv3[2] = ls;
  ASSERT_TRUE(dv3 == hv3);
}

static void TestDevicePointer() {
  g_test = "DevicePointerManipulation";
  {
    thrust::device_vector<int> data(5);
    thrust::device_ptr<int> begin(&data[0]);
    thrust::device_ptr<int> end(&data[0] + 5);
    ASSERT_EQUAL(end - begin, 5);
    begin++;
    begin--;
    ASSERT_EQUAL(end - begin, 5);
    begin += 1;
    begin -= 1;
    ASSERT_EQUAL(end - begin, 5);
    begin = begin + (int)1;
    begin = begin - (int)1;
    ASSERT_EQUAL(end - begin, 5);
    begin = begin + (unsigned int)1;
    begin = begin - (unsigned int)1;
    ASSERT_EQUAL(end - begin, 5);
    begin = begin + (size_t)1;
    begin = begin - (size_t)1;
    ASSERT_EQUAL(end - begin, 5);
    begin = begin + (ptrdiff_t)1;
    begin = begin - (ptrdiff_t)1;
    ASSERT_EQUAL(end - begin, 5);
    begin = begin + (thrust::device_ptr<int>::difference_type)1;
    begin = begin - (thrust::device_ptr<int>::difference_type)1;
    ASSERT_EQUAL(end - begin, 5);
  }
  g_test = "MakeDevicePointer";
  {
    int* raw_ptr = 0;
    thrust::device_ptr<int> p0 = thrust::device_pointer_cast(raw_ptr);
    ASSERT_EQUAL(thrust::raw_pointer_cast(p0), raw_ptr);
    thrust::device_ptr<int> p1 = thrust::device_pointer_cast(p0);
    ASSERT_EQUAL(p0, p1);
  }
  g_test = "RawPointerCast";
  {
    thrust::device_vector<int> vec(3);
    int* first = thrust::raw_pointer_cast(&vec[0]);
    int* last = thrust::raw_pointer_cast(&vec[3]);
    ASSERT_EQUAL(last - first, 3);
    first = thrust::raw_pointer_cast(&vec.front());
    last = thrust::raw_pointer_cast(&vec.back());
    ASSERT_EQUAL(last - first, 2);
    thrust::host_vector<int> hvec(3);
    int* hfirst = thrust::raw_pointer_cast(&hvec[0]);
    int* hlast = thrust::raw_pointer_cast(&hvec[3]);
    ASSERT_EQUAL(hlast - hfirst, 3);
  }
  g_test = "DevicePointerNullptrCompatibility / BoolConversion";
  {
    thrust::device_ptr<double> p0(nullptr);
    ASSERT_TRUE(nullptr == p0);
    ASSERT_TRUE(p0 == nullptr);
    p0 = nullptr;
    ASSERT_TRUE(nullptr == p0);
    ASSERT_TRUE(p0 == nullptr);
    const bool b = bool(p0);
    ASSERT_EQUAL(false, b);
    thrust::device_vector<double> one(1);
    thrust::device_ptr<double> p1 = one.data();
    ASSERT_TRUE(p1 != nullptr);
    ASSERT_TRUE(nullptr != p1);
    ASSERT_EQUAL(true, bool(p1));
  }
}

static void TestDeviceReference() {
  typedef int T;
  g_test = "DeviceReferenceConstructorFromDeviceReference";
  {
    thrust::device_vector<T> v(1, 0);
    thrust::device_reference<T> ref = v[0];
    ASSERT_EQUAL(v[0], ref);
    ASSERT_EQUAL(&v[0], &ref);
    v[0] = 13;
    ASSERT_EQUAL(13, ref);
    ASSERT_EQUAL(v[0], ref);
    ref = 7;
    ASSERT_EQUAL(7, v[0]);
    ASSERT_EQUAL(v[0], ref);
  }
  g_test = "DeviceReferenceConstructorFromDevicePointer";
  {
    thrust::device_vector<T> v(1, 0);
    thrust::device_ptr<T> ptr = &v[0];
    thrust::device_reference<T> ref(ptr);
    ASSERT_EQUAL(*ptr, ref);
    ASSERT_EQUAL(ptr, &ref);
    *ptr = 13;
    ASSERT_EQUAL(13, ref);
    ASSERT_EQUAL(v[0], ref);
    ref = 7;
    ASSERT_EQUAL(7, *ptr);
    ASSERT_EQUAL(v[0], ref);
  }
  g_test = "DeviceReferenceAssignmentFromDeviceReference";
  {
    thrust::device_vector<int> v0(2, 0);
    thrust::device_reference<int> ref0 = v0[0];
    thrust::device_reference<int> ref1 = v0[1];
    ref0 = 13;
    ref1 = ref0;
    ASSERT_EQUAL(13, ref1);
    ASSERT_EQUAL(ref0, ref1);
    thrust::device_vector<float> v1(1, 0.0f);
    thrust::device_reference<float> ref2 = v1[0];
    ref2 = ref1;
    ASSERT_EQUAL(13.0f, ref2);
    ASSERT_EQUAL(ref0, ref2);
    ASSERT_EQUAL(ref1, ref2);
  }
  g_test = "DeviceReferenceManipulation";
  {
    thrust::device_vector<T> v(1, 0);
    thrust::device_ptr<T> ptr = &v[0];
    thrust::device_reference<T> ref(ptr);
#define CHECK_ALL(x) do { ASSERT_EQUAL(x, ref); ASSERT_EQUAL(x, *ptr); ASSERT_EQUAL(x, v[0]); } while (0)
    ref = 0; ++ref; CHECK_ALL(1);
    ref = 0;
    T x1 = ref++;
    ASSERT_EQUAL(0, x1);
    CHECK_ALL(1);
    ref = 0; ref += 5; CHECK_ALL(5);
    ref = 0; --ref; CHECK_ALL(-1);
    ref = 0;
    T x2 = ref--;
    ASSERT_EQUAL(0, x2);
    CHECK_ALL(-1);
    ref = 0; ref -= 5; CHECK_ALL(-5);
    ref = 1; ref *= 5; CHECK_ALL(5);
    ref = 5; ref /= 5; CHECK_ALL(1);
    ref = 5; ref %= 5; CHECK_ALL(0);
    ref = 1; ref <<= 1; CHECK_ALL(2);
    ref = 2; ref >>= 1; CHECK_ALL(1);
    ref = 0; ref |= 1; CHECK_ALL(1);
    ref = 1; ref ^= 1; CHECK_ALL(0);
    ref = 3; ref &= 2; CHECK_ALL(2);
#undef CHECK_ALL
    thrust::device_reference<const T> ref1 = v[0];
    ASSERT_EQUAL(true, ref1 == ref);
  }
  g_test = "DeviceReferenceSwap";
  {
    thrust::device_vector<T> v(2);
    thrust::device_reference<T> ref1 = v.front();
    thrust::device_reference<T> ref2 = v.back();
    ref1 = 7;
    ref2 = 13;
    thrust::swap(ref1, ref2);
    ASSERT_EQUAL(13, ref1);
    ASSERT_EQUAL(7, ref2);
    ref1.swap(ref2);
    ASSERT_EQUAL(7, ref1);
    ASSERT_EQUAL(13, ref2);
  }
}

int main() {
  VectorBasics<thrust::host_vector<int> >();
  VectorBasics<thrust::device_vector<int> >();
  VectorBasics<thrust::device_vector<signed char> >();
  VectorBasics<thrust::device_vector<short> >();
  VectorBasics<thrust::device_vector<long long> >();
  VectorBasics<thrust::device_vector<float> >();
  VectorBasics<thrust::device_vector<double> >();
  VectorInsertSimple<thrust::host_vector<int> >();
  VectorInsertSimple<thrust::device_vector<int> >();
  VectorInsertSimple<thrust::device_vector<unsigned char> >();
  VectorInsertSimple<thrust::device_vector<short> >();
  VectorInsertSimple<thrust::device_vector<unsigned long long> >();
  VectorInsertSimple<thrust::device_vector<float> >();
  VectorInsertSimple<thrust::device_vector<double> >();
  VectorInsertRandom<int>(1);
  VectorInsertRandom<unsigned short>(2);
  VectorInsertRandom<long long>(3);
  for (size_t n : {(size_t)0, (size_t)1, (size_t)63, (size_t)1000, (size_t)10027}) {
    VectorManipulation<thrust::host_vector<int> >(n, 5);
    VectorManipulation<thrust::device_vector<int> >(n, 6);
    VectorManipulation<thrust::device_vector<short> >(n, 7);
    VectorManipulation<thrust::device_vector<double> >(n, 8);
  }
  TestVectorBool();
  TestVectorEqualityAndInequality();
  TestVectorContainingLargeType();
  TestDevicePointer();
  TestDeviceReference();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
