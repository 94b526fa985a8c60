// Front-end test compiled with hipcc: thrust::sort / stable_sort / sort_by_key with user
// comparators and a struct key take the comparison (merge sort) path, whose kernels are
// instantiated in this translation unit.  Known answers are the reference's:
// testing/stable_sort.cu:49-90 (less_div_10), :125-173 (comparator with an external table),
// testing/stable_sort_by_key.cu:50-95; the rest is the reference's host-against-device
// differential pattern (testing/stable_sort.cu:93-108) over its size list.  merge and the
// set operations with user comparators follow: testing/merge.cu:11-38, set_difference.cu:70-90,
// set_intersection.cu:71-91, set_symmetric_difference.cu:70-90, set_union.cu:71-116,
// set_union_by_key.cu:89-120, set_intersection_by_key.cu:83-112.
#include <thrust/device_vector.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/merge.h>
#include <thrust/set_operations.h>
#include <thrust/sort.h>

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
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
struct less_div_10 {
  __host__ __device__ bool operator()(const T& lhs, const T& rhs) const { return ((int)lhs) / 10 < ((int)rhs) / 10; }
};
template <typename T>
struct comp_mod3 {
  const T* table;
  __host__ __device__ bool operator()(T a, T b) const { return table[(int)a] < table[(int)b]; }
};
template <typename T>
struct my_greater {
  __host__ __device__ bool operator()(const T& a, const T& b) const { return b < a; }
};

struct Record {  // a key that is not arithmetic
  int group;
  float weight;
  __host__ __device__ bool operator==(const Record& o) const { return group == o.group && weight == o.weight; }
};
struct by_group_then_heavier {
  __host__ __device__ bool operator()(const Record& a, const Record& b) const {
    return a.group != b.group ? a.group < b.group : b.weight < a.weight;
  }
};
struct by_group {
  __host__ __device__ bool operator()(const Record& a, const Record& b) const { return a.group < b.group; }
};

static const size_t kSizes[] = {0, 1, 2, 3, 15, 16, 17, 31, 32, 33, 255, 256, 257, 1023, 1024, 1025, 4095, 4096, 4097,
                                8191, 8192, 8193, 12293, 16384, 20485, 65533, 65536, 65539, 300007};

static void TestKnownAnswers() {
  g_test = "StableSortSimple";
  thrust::device_vector<int> keys(hv<int>({25, 14, 35, 16, 26, 34, 36, 24, 15}));
  thrust::stable_sort(keys.begin(), keys.end(), less_div_10<int>());
  ASSERT_TRUE(same(to_host(keys), hv<int>({14, 16, 15, 25, 26, 24, 35, 34, 36})));

  g_test = "StableSortByKeySimple";
  thrust::device_vector<int> k2(hv<int>({25, 14, 35, 16, 26, 34, 36, 24, 15}));
  thrust::device_vector<int> v2(hv<int>({0, 1, 2, 3, 4, 5, 6, 7, 8}));
  thrust::stable_sort_by_key(k2.begin(), k2.end(), v2.begin(), less_div_10<int>());
  ASSERT_TRUE(same(to_host(k2), hv<int>({14, 16, 15, 25, 26, 24, 35, 34, 36})));
  ASSERT_TRUE(same(to_host(v2), hv<int>({1, 3, 8, 0, 4, 7, 2, 5, 6})));

  g_test = "StableSortWithIndirection";
  thrust::device_vector<int> data(hv<int>({1, 3, 5, 3, 0, 2, 1}));
  thrust::device_vector<int> table(hv<int>({0, 1, 2, 0, 1, 2}));
  thrust::stable_sort(data.begin(), data.end(), comp_mod3<int>{thrust::raw_pointer_cast(table.data())});
  ASSERT_TRUE(same(to_host(data), hv<int>({3, 3, 0, 1, 1, 5, 2})));

  g_test = "SortWithUserGreater";
  thrust::device_vector<int> d(hv<int>({1, 3, 6, 5, 2, 0, 4}));
  thrust::sort(thrust::device, d.begin(), d.end(), my_greater<int>());
  ASSERT_TRUE(same(to_host(d), hv<int>({6, 5, 4, 3, 2, 1, 0})));
}

template <typename T>
static void Differential(const char* name) {
  g_test = name;
  for (size_t n : kSizes) {
    thrust::host_vector<T> h(n);
    thrust::host_vector<unsigned> hvls(n);
    for (size_t i = 0; i < n; ++i) {
      h[i] = (T)(mix(17 * n + i) % 201);
      hvls[i] = (unsigned)i;
    }
    thrust::device_vector<T> d(h);
    thrust::stable_sort(h.begin(), h.end(), less_div_10<T>());
    thrust::stable_sort(d.begin(), d.end(), less_div_10<T>());
    ASSERT_TRUE(same(to_host(d), h));

    for (size_t i = 0; i < n; ++i) h[i] = (T)(mix(29 * n + i) % 57);
    d = h;
    thrust::device_vector<unsigned> dv(hvls);
    thrust::sort_by_key(h.begin(), h.end(), hvls.begin(), my_greater<T>());
    thrust::sort_by_key(d.begin(), d.end(), dv.begin(), my_greater<T>());
    ASSERT_TRUE(same(to_host(d), h));
    ASSERT_TRUE(same(to_host(dv), hvls));
  }
}

static void TestStructKeys() {
  g_test = "StructKeys";
  for (size_t n : kSizes) {
    std::vector<Record> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = Record{(int)(mix(i + 3 * n) % 23), (float)(mix(i + 7 * n) % 1000) / 8.0f};
    Record* dptr = nullptr;
    unsigned long long* dval = nullptr;
    if (n) {
      dptr = thrust::raw_pointer_cast(thrust::device_malloc<Record>(n));
      dval = thrust::raw_pointer_cast(thrust::device_malloc<unsigned long long>(n));
    }
    std::vector<unsigned long long> hval(n);
    for (size_t i = 0; i < n; ++i) hval[i] = i;
    if (n) {
      (void)hipMemcpy(dptr, h.data(), n * sizeof(Record), hipMemcpyHostToDevice);
      (void)hipMemcpy(dval, hval.data(), n * sizeof(unsigned long long), hipMemcpyHostToDevice);
    }
    // total order on the struct
    thrust::sort(thrust::device, dptr, dptr + n, by_group_then_heavier());
    std::vector<Record> want(h);
    std::stable_sort(want.begin(), want.end(), by_group_then_heavier());
    std::vector<Record> got(n);
    if (n) (void)hipMemcpy(got.data(), dptr, n * sizeof(Record), hipMemcpyDeviceToHost);
    ASSERT_TRUE(same(got, want));
    // a partial order with 8-byte values: stability decides
    if (n) (void)hipMemcpy(dptr, h.data(), n * sizeof(Record), hipMemcpyHostToDevice);
    thrust::stable_sort_by_key(thrust::device, dptr, dptr + n, dval, by_group());
    std::vector<size_t> order(n);
    for (size_t i = 0; i < n; ++i) order[i] = i;
    std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) { return h[a].group < h[b].group; });
    std::vector<unsigned long long> gotv(n);
    if (n) {
      (void)hipMemcpy(got.data(), dptr, n * sizeof(Record), hipMemcpyDeviceToHost);
      (void)hipMemcpy(gotv.data(), dval, n * sizeof(unsigned long long), hipMemcpyDeviceToHost);
    }
    bool ok = true;
    for (size_t i = 0; i < n; ++i) ok = ok && got[i] == h[order[i]] && gotv[i] == order[i];
    ASSERT_TRUE(ok);
    if (n) {
      thrust::device_free(thrust::device_pointer_cast(dptr));
      thrust::device_free(thrust::device_pointer_cast(dval));
    }
  }
}

template <typename T>
struct my_less {
  __host__ __device__ bool operator()(const T& a, const T& b) const { return a < b; }
};

static void TestMergeWithUserComparators() {
  g_test = "MergeSimple";  // testing/merge.cu:11-38 and merge_by_key.cu:10-45 through a user-defined less
  {
    thrust::device_vector<int> a(hv<int>({0, 2, 4})), b(hv<int>({0, 3, 3, 4})), out(7);
    auto end = thrust::merge(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less<int>());
    ASSERT_TRUE(end - out.begin() == 7);
    ASSERT_TRUE(same(to_host(out), hv<int>({0, 0, 2, 3, 3, 4, 4})));
    thrust::device_vector<int> va(hv<int>({13, 7, 42})), vb(hv<int>({42, 42, 7, 13})), ko(7), vo(7);
    auto ends = thrust::merge_by_key(a.begin(), a.end(), b.begin(), b.end(), va.begin(), vb.begin(), ko.begin(),
                                     vo.begin(), my_less<int>());
    ASSERT_TRUE(ends.first - ko.begin() == 7 && ends.second - vo.begin() == 7);
    ASSERT_TRUE(same(to_host(ko), hv<int>({0, 0, 2, 3, 3, 4, 4})));
    ASSERT_TRUE(same(to_host(vo), hv<int>({13, 42, 7, 42, 7, 42, 13})));  // ties: the first range first
  }
  g_test = "MergeDifferential";
  for (size_t n : kSizes) {
    const size_t na = n, nb = n / 3 + (n % 5);
    thrust::host_vector<int> ha(na), hb(nb);
    for (size_t i = 0; i < na; ++i) ha[i] = (int)(mix(i + 11 * n) % 997);
    for (size_t i = 0; i < nb; ++i) hb[i] = (int)(mix(i + 13 * n) % 997);
    // equivalence classes of ten under less_div_10; inside a class the input order must survive
    std::stable_sort(ha.begin(), ha.end(), less_div_10<int>());
    std::stable_sort(hb.begin(), hb.end(), less_div_10<int>());
    thrust::device_vector<int> da(ha), db(hb), dout(na + nb);
    thrust::host_vector<int> hout(na + nb);
    thrust::merge(ha.begin(), ha.end(), hb.begin(), hb.end(), hout.begin(), less_div_10<int>());
    thrust::merge(da.begin(), da.end(), db.begin(), db.end(), dout.begin(), less_div_10<int>());
    ASSERT_TRUE(same(to_host(dout), hout));
    // descending with values
    std::stable_sort(ha.begin(), ha.end(), my_greater<int>());
    std::stable_sort(hb.begin(), hb.end(), my_greater<int>());
    da = ha;
    db = hb;
    thrust::host_vector<unsigned> hva(na), hvb(nb), hvo(na + nb);
    for (size_t i = 0; i < na; ++i) hva[i] = (unsigned)i;
    for (size_t i = 0; i < nb; ++i) hvb[i] = (unsigned)(1000000 + i);
    thrust::device_vector<unsigned> dva(hva), dvb(hvb), dvo(na + nb);
    thrust::merge_by_key(ha.begin(), ha.end(), hb.begin(), hb.end(), hva.begin(), hvb.begin(), hout.begin(), hvo.begin(),
                         my_greater<int>());
    thrust::merge_by_key(da.begin(), da.end(), db.begin(), db.end(), dva.begin(), dvb.begin(), dout.begin(), dvo.begin(),
                         my_greater<int>());
    ASSERT_TRUE(same(to_host(dout), hout));
    ASSERT_TRUE(same(to_host(dvo), hvo));
  }
}

static void TestSetOperationsWithUserComparators() {
  g_test = "SetOperationsSimple";
  {
    thrust::device_vector<int> a(hv<int>({0, 2, 4, 5})), b(hv<int>({0, 3, 3, 4, 6})), out(9);
    auto end = thrust::set_difference(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less<int>());
    ASSERT_TRUE(end - out.begin() == 2);
    out.resize(2);
    ASSERT_TRUE(same(to_host(out), hv<int>({2, 5})));
  }
  {
    thrust::device_vector<int> a(hv<int>({0, 2, 4})), b(hv<int>({0, 3, 3, 4})), out(7);
    auto end = thrust::set_intersection(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less<int>());
    ASSERT_TRUE(end - out.begin() == 2);
    out.resize(2);
    ASSERT_TRUE(same(to_host(out), hv<int>({0, 4})));
    out.resize(7);
    end = thrust::set_union(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less<int>());
    ASSERT_TRUE(end - out.begin() == 5);
    out.resize(5);
    ASSERT_TRUE(same(to_host(out), hv<int>({0, 2, 3, 3, 4})));
    // by key: a tie takes the first range's value; the second range's surplus keeps its own
    thrust::device_vector<int> va(hv<int>({0, 0, 0})), vb(hv<int>({1, 1, 1, 1})), ko(7), vo(7);
    auto ends = thrust::set_union_by_key(a.begin(), a.end(), b.begin(), b.end(), va.begin(), vb.begin(), ko.begin(),
                                         vo.begin(), my_less<int>());
    ASSERT_TRUE(ends.first - ko.begin() == 5 && ends.second - vo.begin() == 5);
    ko.resize(5);
    vo.resize(5);
    ASSERT_TRUE(same(to_host(ko), hv<int>({0, 2, 3, 3, 4})));
    ASSERT_TRUE(same(to_host(vo), hv<int>({0, 0, 1, 1, 0})));
    ko.resize(7);
    vo.resize(7);
    ends = thrust::set_intersection_by_key(a.begin(), a.end(), b.begin(), b.end(), va.begin(), ko.begin(), vo.begin(),
                                           my_less<int>());
    ASSERT_TRUE(ends.first - ko.begin() == 2 && ends.second - vo.begin() == 2);
    ko.resize(2);
    vo.resize(2);
    ASSERT_TRUE(same(to_host(ko), hv<int>({0, 4})));
    ASSERT_TRUE(same(to_host(vo), hv<int>({0, 0})));
  }
  {
    thrust::device_vector<int> a(hv<int>({0, 2, 2})), b(hv<int>({0, 2, 2, 2, 3})), out(8);
    auto end = thrust::set_union(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less<int>());
    ASSERT_TRUE(end - out.begin() == 5);
    out.resize(5);
    ASSERT_TRUE(same(to_host(out), hv<int>({0, 2, 2, 2, 3})));
  }
  {
    thrust::device_vector<int> a(hv<int>({0, 2, 4, 6})), b(hv<int>({0, 3, 3, 4, 7})), out(9);
    auto end = thrust::set_symmetric_difference(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less<int>());
    ASSERT_TRUE(end - out.begin() == 5);
    out.resize(5);
    ASSERT_TRUE(same(to_host(out), hv<int>({2, 3, 3, 6, 7})));
  }
  g_test = "SetOperationsDifferential";
  for (size_t n : kSizes) {
    const size_t na = n, nb = n / 2 + (n % 7);
    // equivalence classes of ten under less_div_10, a few dozen elements in each for the
    // larger sizes: which copies survive shows in the low digit
    const uint64_t range = n < 64 ? 40 : (n < 5000 ? 400 : 3000);
    thrust::host_vector<int> ha(na), hb(nb);
    for (size_t i = 0; i < na; ++i) ha[i] = (int)(mix(i + 17 * n) % range);
    for (size_t i = 0; i < nb; ++i) hb[i] = (int)(mix(i + 19 * n) % range);
    std::stable_sort(ha.begin(), ha.end(), less_div_10<int>());
    std::stable_sort(hb.begin(), hb.end(), less_div_10<int>());
    thrust::host_vector<unsigned> hva(na), hvb(nb);
    for (size_t i = 0; i < na; ++i) hva[i] = (unsigned)i;
    for (size_t i = 0; i < nb; ++i) hvb[i] = (unsigned)(1000000 + i);
    thrust::device_vector<int> da(ha), db(hb);
    thrust::device_vector<unsigned> dva(hva), dvb(hvb);
    thrust::host_vector<int> hout(na + nb);
    thrust::device_vector<int> dout(na + nb);
    thrust::host_vector<unsigned> hvo(na + nb);
    thrust::device_vector<unsigned> dvo(na + nb);
    const less_div_10<int> comp;
    size_t hc, dc;
#define CHECK_KEYS(NAME)                                                                                   \
    hc = thrust::NAME(ha.begin(), ha.end(), hb.begin(), hb.end(), hout.begin(), comp) - hout.begin();      \
    dc = thrust::NAME(da.begin(), da.end(), db.begin(), db.end(), dout.begin(), comp) - dout.begin();      \
    ASSERT_TRUE(hc == dc);                                                                                 \
    {                                                                                                      \
      thrust::host_vector<int> got(dout);                                                                  \
      ASSERT_TRUE(std::equal(hout.begin(), hout.begin() + hc, got.begin()));                               \
    }
    CHECK_KEYS(set_difference)
    CHECK_KEYS(set_intersection)
    CHECK_KEYS(set_symmetric_difference)
    CHECK_KEYS(set_union)
#undef CHECK_KEYS
#define CHECK_BY_KEY(NAME)                                                                                 \
    hc = thrust::NAME(ha.begin(), ha.end(), hb.begin(), hb.end(), hva.begin(), hvb.begin(), hout.begin(),  \
                      hvo.begin(), comp).first - hout.begin();                                             \
    dc = thrust::NAME(da.begin(), da.end(), db.begin(), db.end(), dva.begin(), dvb.begin(), dout.begin(),  \
                      dvo.begin(), comp).first - dout.begin();                                             \
    ASSERT_TRUE(hc == dc);                                                                                 \
    {                                                                                                      \
      thrust::host_vector<int> got(dout);                                                                  \
      thrust::host_vector<unsigned> got_values(dvo);                                                       \
      ASSERT_TRUE(std::equal(hout.begin(), hout.begin() + hc, got.begin()));                               \
      ASSERT_TRUE(std::equal(hvo.begin(), hvo.begin() + hc, got_values.begin()));                          \
    }
    CHECK_BY_KEY(set_difference_by_key)
    CHECK_BY_KEY(set_symmetric_difference_by_key)
    CHECK_BY_KEY(set_union_by_key)
#undef CHECK_BY_KEY
    hc = thrust::set_intersection_by_key(ha.begin(), ha.end(), hb.begin(), hb.end(), hva.begin(), hout.begin(),
                                         hvo.begin(), comp).first - hout.begin();
    dc = thrust::set_intersection_by_key(da.begin(), da.end(), db.begin(), db.end(), dva.begin(), dout.begin(),
                                         dvo.begin(), comp).first - dout.begin();
    ASSERT_TRUE(hc == dc);
    {
      thrust::host_vector<int> got(dout);
      thrust::host_vector<unsigned> got_values(dvo);
      ASSERT_TRUE(std::equal(hout.begin(), hout.begin() + hc, got.begin()));
      ASSERT_TRUE(std::equal(hvo.begin(), hvo.begin() + hc, got_values.begin()));
    }
  }
  g_test = "SetOperationsStructKeys";
  {
    // records ordered by group only: the weight tells which copies were kept
    const size_t na = 5000, nb = 3000;
    thrust::host_vector<Record> ha(na), hb(nb);
    for (size_t i = 0; i < na; ++i) ha[i] = Record{(int)(mix(i + 5) % 700), (float)i};
    for (size_t i = 0; i < nb; ++i) hb[i] = Record{(int)(mix(i + 7) % 700), -(float)i};
    std::stable_sort(ha.begin(), ha.end(), by_group());
    std::stable_sort(hb.begin(), hb.end(), by_group());
    thrust::device_vector<Record> da(ha), db(hb), dout(na + nb);
    thrust::host_vector<Record> hout(na + nb);
    size_t hc = thrust::set_union(ha.begin(), ha.end(), hb.begin(), hb.end(), hout.begin(), by_group()) - hout.begin();
    size_t dc = thrust::set_union(da.begin(), da.end(), db.begin(), db.end(), dout.begin(), by_group()) - dout.begin();
    ASSERT_TRUE(hc == dc);
    thrust::host_vector<Record> got(dout);
    ASSERT_TRUE(std::equal(hout.begin(), hout.begin() + hc, got.begin()));
    hc = thrust::set_difference(ha.begin(), ha.end(), hb.begin(), hb.end(), hout.begin(), by_group()) - hout.begin();
    dc = thrust::set_difference(da.begin(), da.end(), db.begin(), db.end(), dout.begin(), by_group()) - dout.begin();
    ASSERT_TRUE(hc == dc);
    got = dout;
    ASSERT_TRUE(std::equal(hout.begin(), hout.begin() + hc, got.begin()));
  }
}

int main() {
  TestKnownAnswers();
  Differential<signed char>("signed char");
  Differential<short>("short");
  Differential<int>("int");
  Differential<long long>("long long");
  Differential<float>("float");
  TestStructKeys();
  TestMergeWithUserComparators();
  TestSetOperationsWithUserComparators();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
