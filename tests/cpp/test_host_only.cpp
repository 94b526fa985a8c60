// Host-system behaviour that needs no GPU: run by tests/test_host_system.py on any machine.
// Each expectation is what the reference's sequential system produces for the same call.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include <thrust/adjacent_difference.h>
#include <thrust/binary_search.h>
#include <thrust/equal.h>
#include <thrust/extrema.h>
#include <thrust/find.h>
#include <thrust/iterator/reverse_iterator.h>
#include <thrust/logical.h>
#include <thrust/mismatch.h>
#include <thrust/partition.h>
#include <thrust/replace.h>
#include <thrust/reverse.h>
#include <thrust/sort.h>
#include <thrust/swap.h>
#include <thrust/tabulate.h>
#include <thrust/uninitialized_copy.h>
#include <thrust/uninitialized_fill.h>
#include <thrust/device_free.h>
#include <thrust/device_malloc.h>
#include <thrust/device_reference.h>
#include <thrust/distance.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/reduce.h>
#include <thrust/sort.h>

static int g_checks = 0, g_fail = 0;
#define CHECK(c)                                                          \
  do {                                                                    \
    ++g_checks;                                                           \
    if (!(c)) { ++g_fail; std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #c); } \
  } while (0)

struct within_one {
  bool operator()(int a, int b) const { return std::abs(a - b) <= 1; }
};

// thrust/system/detail/sequential/reduce_by_key.h:61-87: a run lasts while pred(first key of
// the run, key) holds.  A predicate that is not transitive tells this from a comparison of
// neighbours: 1 2 3 4 is two runs (1 2 | 3 4), not one.
static void TestReduceByKeyComparesWithTheRunsFirstKey() {
  thrust::host_vector<int> keys(std::vector<int>{1, 2, 3, 4, 4, 6, 7, 8});
  thrust::host_vector<int> vals(std::vector<int>{1, 10, 100, 1000, 10000, 100000, 1000000, 10000000});
  thrust::host_vector<int> ko(8), vo(8);
  auto ends = thrust::reduce_by_key(thrust::host, keys.begin(), keys.end(), vals.begin(), ko.begin(), vo.begin(),
                                    within_one(), thrust::plus<int>());
  CHECK(ends.first - ko.begin() == 4);
  CHECK(ko[0] == 1 && vo[0] == 11);
  CHECK(ko[1] == 3 && vo[1] == 11100);
  CHECK(ko[2] == 6 && vo[2] == 1100000);
  CHECK(ko[3] == 8 && vo[3] == 10000000);
}

// thrust/system/detail/sequential/sort.inl:139-148: less<K> / greater<K> on arithmetic keys take
// the radix sort, which orders floats by their bits; any other comparator takes the merge
// sort, for which -0.0 and +0.0 are equivalent and keep their order.
static void TestFloatZerosUnderLessAndUnderAUserComparator() {
  const float pz = 0.0f, nz = -0.0f;
  thrust::host_vector<float> k(std::vector<float>{pz, nz, 1.0f, pz, nz, -1.0f});
  thrust::host_vector<int> v(std::vector<int>{0, 1, 2, 3, 4, 5});
  thrust::host_vector<float> k1 = k;
  thrust::host_vector<int> v1 = v;
  thrust::stable_sort_by_key(thrust::host, k1.begin(), k1.end(), v1.begin(), thrust::less<float>());
  const int want_less[] = {5, 1, 4, 0, 3, 2};
  for (int i = 0; i < 6; ++i) CHECK(v1[i] == want_less[i]);
  CHECK(std::signbit(k1[1]) && std::signbit(k1[2]) && !std::signbit(k1[3]) && !std::signbit(k1[4]));

  thrust::host_vector<float> k2 = k;
  thrust::host_vector<int> v2 = v;
  thrust::stable_sort_by_key(thrust::host, k2.begin(), k2.end(), v2.begin(), thrust::greater<float>());
  const int want_greater[] = {2, 0, 3, 1, 4, 5};
  for (int i = 0; i < 6; ++i) CHECK(v2[i] == want_greater[i]);

  thrust::host_vector<float> k3 = k;
  thrust::host_vector<int> v3 = v;
  thrust::stable_sort_by_key(thrust::host, k3.begin(), k3.end(), v3.begin(),
                             [](float a, float b) { return a < b; });
  const int want_user[] = {5, 0, 1, 3, 4, 2};
  for (int i = 0; i < 6; ++i) CHECK(v3[i] == want_user[i]);
}

// thrust/functional.h:420-1493 in the reference: the arithmetic, bitwise and logical functors,
// the projections and the negators, here through host algorithms.
static void TestFunctors() {
  thrust::host_vector<unsigned> x(std::vector<unsigned>{12, 10, 7, 5});
  CHECK(thrust::reduce(thrust::host, x.begin(), x.end(), 0u, thrust::bit_xor<unsigned>()) == (12u ^ 10u ^ 7u ^ 5u));
  CHECK(thrust::reduce(thrust::host, x.begin(), x.end(), ~0u, thrust::bit_and<unsigned>()) == (12u & 10u & 7u & 5u));
  CHECK(thrust::reduce(thrust::host, x.begin(), x.end(), 0u, thrust::bit_or<unsigned>()) == 15u);
  CHECK(thrust::divides<int>()(17, 5) == 3 && thrust::modulus<int>()(17, 5) == 2);
  CHECK(thrust::divides<>()(9.0, 2) == 4.5);
  CHECK(thrust::logical_and<int>()(3, 0) == false && thrust::logical_or<int>()(3, 0) == true);
  CHECK(thrust::logical_not<>()(0) == true);
  CHECK((thrust::project1st<int, double>()(4, 2.5) == 4) && (thrust::project2nd<int, double>()(4, 2.5) == 2.5));
  CHECK(thrust::project2nd<>()(4, 'c') == 'c');
  CHECK(thrust::reduce(thrust::host, x.begin(), x.end(), 99u, thrust::project2nd<unsigned, unsigned>()) == 5u);
  CHECK(thrust::not2(within_one())(1, 2) == false && thrust::not2(within_one())(1, 3) == true);
  struct is_odd { bool operator()(unsigned v) const { return v & 1u; } };
  CHECK(thrust::not1(is_odd())(12u) == true && thrust::not1(is_odd())(7u) == false);
}

static void TestDistance() {
  thrust::host_vector<int> v(17);
  CHECK(thrust::distance(v.begin(), v.end()) == 17);
  thrust::device_ptr<int> p(nullptr);
  CHECK(thrust::distance(p, p + 5) == 5);
}

// The callers around the path on the host system, in a translation unit compiled by g++: the
// reference's vectors (testing/min_element.cu:6-30, find.cu:44-60, is_sorted.cu:6-40,
// binary_search.cu:50-90, adjacent_difference.cu:6-40, replace.cu:6-40, reverse.cu:6-40, tabulate.cu:6-40).
static void TestCallersAroundThePath() {
  thrust::host_vector<int> v(6), w(6);
  v[0] = 3; v[1] = 5; v[2] = 1; v[3] = 2; v[4] = 5; v[5] = 1;
  CHECK(thrust::min_element(v.begin(), v.end()) - v.begin() == 2);
  CHECK(thrust::max_element(thrust::host, v.begin(), v.end()) - v.begin() == 1);
  CHECK(thrust::minmax_element(v.begin(), v.end()).second - v.begin() == 1);
  CHECK(thrust::find(v.begin(), v.end(), 2) - v.begin() == 3);
  CHECK(thrust::find(v.begin(), v.end(), 7) == v.end());
  CHECK(thrust::any_of(v.begin(), v.end(), thrust::identity<int>()));
  CHECK(thrust::all_of(v.begin(), v.end(), thrust::identity<int>()));
  CHECK(!thrust::none_of(v.begin(), v.end(), thrust::identity<int>()));
  CHECK(!thrust::is_sorted(v.begin(), v.end()));
  CHECK(thrust::is_sorted_until(v.begin(), v.end()) - v.begin() == 2);
  thrust::sort(v.begin(), v.end());  // 1 1 2 3 5 5
  CHECK(thrust::is_sorted(v.begin(), v.end()));
  CHECK(thrust::lower_bound(v.begin(), v.end(), 5) - v.begin() == 4);
  CHECK(thrust::upper_bound(v.begin(), v.end(), 1) - v.begin() == 2);
  CHECK(thrust::binary_search(v.begin(), v.end(), 3) && !thrust::binary_search(v.begin(), v.end(), 4));
  CHECK(thrust::equal_range(v.begin(), v.end(), 5).second == v.end());
  thrust::adjacent_difference(v.begin(), v.end(), w.begin());
  CHECK(w[0] == 1 && w[1] == 0 && w[2] == 1 && w[3] == 1 && w[4] == 2 && w[5] == 0);
  thrust::reverse(v.begin(), v.end());
  CHECK(v[0] == 5 && v[5] == 1);
  thrust::replace(v.begin(), v.end(), 5, 9);
  CHECK(v[0] == 9 && v[1] == 9 && v[2] == 3);
  CHECK(thrust::equal(v.begin(), v.end(), v.begin()) && !thrust::equal(v.begin(), v.end(), w.begin()));
  CHECK(thrust::mismatch(v.begin(), v.end(), w.begin()).first == v.begin());
  thrust::swap_ranges(v.begin(), v.end(), w.begin());
  CHECK(w[0] == 9 && v[0] == 1);
  thrust::tabulate(v.begin(), v.end(), thrust::negate<std::ptrdiff_t>());
  CHECK(v[2] == -2 && v[5] == -5);
  CHECK(*thrust::make_reverse_iterator(v.end()) == -5);
  CHECK(thrust::partition_point(w.begin(), w.end(), thrust::identity<int>()) == w.end());
  CHECK(thrust::is_partitioned(w.begin(), w.end(), thrust::identity<int>()));
  thrust::uninitialized_fill(v.begin(), v.end(), 4);
  thrust::uninitialized_copy(v.begin(), v.begin() + 2, w.begin());
  CHECK(w[0] == 4 && w[1] == 4 && w[2] == 3);
}

int main() {
  TestCallersAroundThePath();
  TestFunctors();
  TestDistance();
  TestReduceByKeyComparesWithTheRunsFirstKey();
  TestFloatZerosUnderLessAndUnderAUserComparator();
  std::printf("%d checks, %d failed\n", g_checks, g_fail);
  return g_fail ? 1 : 0;
}
