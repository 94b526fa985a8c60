// The paths that run in kernels instantiated in the user's translation unit -- user-defined
// operators, predicates, key equalities and comparators through the thrust:: front end --
// beside the same job done with the library's own functors (thrust::plus, thrust::equal_to,
// placeholder predicates, thrust::less), which goes through libthrust_amd.so's entry points.
// Every pair must produce the same output (checked: sizes and contents), and the two times
// are printed side by side.  Every line is the blocking call as a user makes it (temporary
// storage from the caching arena, result sizes copied back), best of five after one warm-up,
// inputs resident in HBM.  Bytes are the algorithmic ones (a range read once, a result
// written once).
//
//   tests/cpp/bin/test_user_functor_paths [log2 of the element count, default 27]
#include <thrust/adjacent_difference.h>
#include <thrust/binary_search.h>
#include <thrust/copy.h>
#include <thrust/device_vector.h>
#include <thrust/extrema.h>
#include <thrust/find.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/merge.h>
#include <thrust/partition.h>
#include <thrust/reduce.h>
#include <thrust/remove.h>
#include <thrust/scan.h>
#include <thrust/set_operations.h>
#include <thrust/sort.h>
#include <thrust/transform.h>
#include <thrust/unique.h>

#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

struct my_plus {
  __host__ __device__ unsigned operator()(unsigned a, unsigned b) const { return a + b; }
};
struct my_less {
  __host__ __device__ bool operator()(unsigned a, unsigned b) const { return a < b; }
};
struct my_equal {
  __host__ __device__ bool operator()(unsigned a, unsigned b) const { return a == b; }
};
struct my_below {
  unsigned limit;
  __host__ __device__ bool operator()(unsigned a) const { return a < limit; }
};
struct scramble {  // a counter-based generator: element i of the inputs
  uint64_t seed;
  __host__ __device__ unsigned operator()(uint64_t i) const {
    uint64_t z = i + seed + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return (unsigned)(z ^ (z >> 31));
  }
};
struct modulo {
  unsigned m;
  __host__ __device__ unsigned operator()(unsigned x) const { return x % m; }
};

template <typename F>
static double best_ms(F f) {
  f();
  double best = 1e30;
  for (int rep = 0; rep < 5; ++rep) {
    (void)hipDeviceSynchronize();
    const auto t0 = std::chrono::steady_clock::now();
    f();
    (void)hipDeviceSynchronize();
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    if (ms < best) best = ms;
  }
  return best;
}
static int g_failed = 0;
static void expect(bool ok, const char* what) {
  if (!ok) {
    ++g_failed;
    std::printf("MISMATCH: %s\n", what);
  }
}
// one job done both ways: time of the user's functor, time of the library's, and their ratio
static void pair_line(const char* what, double user_ms, double lib_ms, double bytes) {
  std::printf("%-34s user %8.3f ms %5.1f%%   library %8.3f ms %5.1f%%   ratio %4.2f\n", what, user_ms,
              bytes / user_ms / 1e6 / 80.0, lib_ms, bytes / lib_ms / 1e6 / 80.0, user_ms / lib_ms);
}
typedef thrust::device_vector<unsigned> dvec;
static bool same_prefix(const dvec& a, const dvec& b, size_t count) {
  const thrust::host_vector<unsigned> ha(a.begin(), a.begin() + count), hb(b.begin(), b.begin() + count);
  return ha == hb;
}

int main(int argc, char** argv) {
  using namespace thrust::placeholders;
  const int lg = argc > 1 ? std::atoi(argv[1]) : 27;
  const size_t n = (size_t)1 << lg;
  std::printf("user functors and the library's own through the front end, n = 2^%d uint32; %% of 8 TB/s\n", lg);
  thrust::counting_iterator<uint64_t> index(0);
  dvec x(n), y(n), out(2 * n), out2(2 * n), vals(n), vout(n), vout2(n), rest(n), rest2(n);
  thrust::copy(thrust::make_transform_iterator(index, scramble{1}), thrust::make_transform_iterator(index, scramble{1}) + n,
               x.begin());
  thrust::copy(thrust::make_transform_iterator(index, scramble{2}), thrust::make_transform_iterator(index, scramble{2}) + n,
               vals.begin());
  unsigned ru = 0, rl = 0;
  double tu, tl;

  tu = best_ms([&] { ru = thrust::reduce(x.begin(), x.end(), 0u, my_plus()); });
  tl = best_ms([&] { rl = thrust::reduce(x.begin(), x.end(), 0u, thrust::plus<unsigned>()); });
  expect(ru == rl, "reduce");
  pair_line("reduce", tu, tl, 4.0 * n);
  tu = best_ms([&] { thrust::inclusive_scan(x.begin(), x.end(), out.begin(), my_plus()); });
  tl = best_ms([&] { thrust::inclusive_scan(x.begin(), x.end(), out2.begin(), thrust::plus<unsigned>()); });
  expect(same_prefix(out, out2, n), "inclusive_scan");
  pair_line("inclusive_scan", tu, tl, 8.0 * n);

  // selection at 50 % and 5 %
  for (unsigned pct : {50u, 5u}) {
    const unsigned limit = (unsigned)(((uint64_t)1 << 32) * pct / 100);
    char name[64];
    size_t cu = 0, cl = 0;
    tu = best_ms([&] { cu = thrust::copy_if(x.begin(), x.end(), out.begin(), my_below{limit}) - out.begin(); });
    tl = best_ms([&] { cl = thrust::copy_if(x.begin(), x.end(), out2.begin(), _1 < limit) - out2.begin(); });
    expect(cu == cl && same_prefix(out, out2, cu), "copy_if");
    std::snprintf(name, sizeof name, "copy_if, %u %% selected", pct);
    pair_line(name, tu, tl, 4.0 * n + 4.0 * cu);
    tu = best_ms([&] { cu = thrust::copy_if(vals.begin(), vals.end(), x.begin(), out.begin(), my_below{limit}) - out.begin(); });
    tl = best_ms([&] { cl = thrust::copy_if(vals.begin(), vals.end(), x.begin(), out2.begin(), _1 < limit) - out2.begin(); });
    expect(cu == cl && same_prefix(out, out2, cu), "copy_if by stencil");
    std::snprintf(name, sizeof name, "copy_if by stencil, %u %%", pct);
    pair_line(name, tu, tl, 8.0 * n + 4.0 * cu);
    tu = best_ms([&] {
      cu = thrust::partition_copy(x.begin(), x.end(), out.begin(), rest.begin(), my_below{limit}).first - out.begin();
    });
    tl = best_ms([&] {
      cl = thrust::partition_copy(x.begin(), x.end(), out2.begin(), rest2.begin(), _1 < limit).first - out2.begin();
    });
    expect(cu == cl && same_prefix(out, out2, cu) && same_prefix(rest, rest2, n - cu), "partition_copy");
    std::snprintf(name, sizeof name, "partition_copy, %u %%", pct);
    pair_line(name, tu, tl, 8.0 * n);
    // in place: every repetition partitions a fresh copy; the copy is timed by itself and taken off
    const double copy_ms = best_ms([&] { thrust::copy(x.begin(), x.end(), out.begin()); });
    tu = best_ms([&] {
      thrust::copy(x.begin(), x.end(), out.begin());
      cu = thrust::stable_partition(out.begin(), out.begin() + n, my_below{limit}) - out.begin();
    }) - copy_ms;
    tl = best_ms([&] {
      thrust::copy(x.begin(), x.end(), out2.begin());
      cl = thrust::stable_partition(out2.begin(), out2.begin() + n, _1 < limit) - out2.begin();
    }) - copy_ms;
    expect(cu == cl && same_prefix(out, out2, n), "stable_partition");
    std::snprintf(name, sizeof name, "stable_partition, %u %%", pct);
    pair_line(name, tu, tl, 8.0 * n);
  }

  // sorted keys with runs of about eight
  thrust::copy(thrust::make_transform_iterator(x.begin(), modulo{(unsigned)(n / 8)}),
               thrust::make_transform_iterator(x.begin(), modulo{(unsigned)(n / 8)}) + n, y.begin());
  thrust::sort(y.begin(), y.end());
  size_t runs = 0, runs2 = 0;
  tu = best_ms([&] { runs = thrust::unique_copy(y.begin(), y.end(), out.begin(), my_equal()) - out.begin(); });
  tl = best_ms([&] { runs2 = thrust::unique_copy(y.begin(), y.end(), out2.begin()) - out2.begin(); });
  expect(runs == runs2 && same_prefix(out, out2, runs), "unique_copy");
  pair_line("unique_copy, mean run 8", tu, tl, 4.0 * n + 4.0 * runs);
  tu = best_ms([&] {
    runs = thrust::unique_by_key_copy(y.begin(), y.end(), vals.begin(), out.begin(), vout.begin(), my_equal()).first - out.begin();
  });
  tl = best_ms([&] {
    runs2 = thrust::unique_by_key_copy(y.begin(), y.end(), vals.begin(), out2.begin(), vout2.begin()).first - out2.begin();
  });
  expect(runs == runs2 && same_prefix(out, out2, runs) && same_prefix(vout, vout2, runs), "unique_by_key_copy");
  pair_line("unique_by_key_copy, mean run 8", tu, tl, 8.0 * n + 8.0 * runs);
  tu = best_ms([&] {
    runs = thrust::reduce_by_key(y.begin(), y.end(), vals.begin(), out.begin(), vout.begin(), my_equal(), my_plus()).first -
           out.begin();
  });
  tl = best_ms([&] {
    runs2 = thrust::reduce_by_key(y.begin(), y.end(), vals.begin(), out2.begin(), vout2.begin(), thrust::equal_to<unsigned>(),
                                  thrust::plus<unsigned>()).first - out2.begin();
  });
  expect(runs == runs2 && same_prefix(out, out2, runs) && same_prefix(vout, vout2, runs), "reduce_by_key");
  pair_line("reduce_by_key, mean run 8", tu, tl, 8.0 * n + 8.0 * runs);
  std::printf("  (%zu runs)\n", runs);
  tu = best_ms([&] { thrust::inclusive_scan_by_key(y.begin(), y.end(), vals.begin(), out.begin(), my_equal(), my_plus()); });
  tl = best_ms([&] {
    thrust::inclusive_scan_by_key(y.begin(), y.end(), vals.begin(), out2.begin(), thrust::equal_to<unsigned>(),
                                  thrust::plus<unsigned>());
  });
  expect(same_prefix(out, out2, n), "inclusive_scan_by_key");
  pair_line("inclusive_scan_by_key, mean run 8", tu, tl, 12.0 * n);
  tu = best_ms([&] { thrust::exclusive_scan_by_key(y.begin(), y.end(), vals.begin(), out.begin(), 7u, my_equal(), my_plus()); });
  tl = best_ms([&] {
    thrust::exclusive_scan_by_key(y.begin(), y.end(), vals.begin(), out2.begin(), 7u, thrust::equal_to<unsigned>(),
                                  thrust::plus<unsigned>());
  });
  expect(same_prefix(out, out2, n), "exclusive_scan_by_key");
  pair_line("exclusive_scan_by_key, mean run 8", tu, tl, 12.0 * n);

  // two sorted ranges of n / 2 with duplicates in and across them
  const size_t m = n / 2;
  dvec a(m), b(m);
  thrust::copy(thrust::make_transform_iterator(x.begin(), modulo{(unsigned)(m / 4)}),
               thrust::make_transform_iterator(x.begin(), modulo{(unsigned)(m / 4)}) + m, a.begin());
  thrust::copy(thrust::make_transform_iterator(x.begin() + m, modulo{(unsigned)(m / 2)}),
               thrust::make_transform_iterator(x.begin() + m, modulo{(unsigned)(m / 2)}) + m, b.begin());
  thrust::sort(a.begin(), a.end());
  thrust::sort(b.begin(), b.end());
  tu = best_ms([&] { thrust::merge(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less()); });
  tl = best_ms([&] { thrust::merge(a.begin(), a.end(), b.begin(), b.end(), out2.begin()); });
  expect(same_prefix(out, out2, n), "merge");
  pair_line("merge", tu, tl, 8.0 * n);
  size_t kept = 0, kept2 = 0;
  tu = best_ms([&] { kept = thrust::set_union(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less()) - out.begin(); });
  tl = best_ms([&] { kept2 = thrust::set_union(a.begin(), a.end(), b.begin(), b.end(), out2.begin()) - out2.begin(); });
  expect(kept == kept2 && same_prefix(out, out2, kept), "set_union");
  pair_line("set_union", tu, tl, 4.0 * n + 4.0 * kept);
  tu = best_ms([&] {
    kept = thrust::set_intersection(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less()) - out.begin();
  });
  tl = best_ms([&] { kept2 = thrust::set_intersection(a.begin(), a.end(), b.begin(), b.end(), out2.begin()) - out2.begin(); });
  expect(kept == kept2 && same_prefix(out, out2, kept), "set_intersection");
  pair_line("set_intersection", tu, tl, 4.0 * n + 4.0 * kept);

  // the sort last: it is in place, every repetition sorts a fresh copy (the copy is timed by itself and
  // taken off).  The user's comparator takes the merge sort, thrust::less the radix sort.
  const double copy_ms = best_ms([&] { thrust::copy(x.begin(), x.end(), out.begin()); });
  tu = best_ms([&] {
    thrust::copy(x.begin(), x.end(), out.begin());
    thrust::sort(out.begin(), out.begin() + n, my_less());
  }) - copy_ms;
  tl = best_ms([&] {
    thrust::copy(x.begin(), x.end(), out2.begin());
    thrust::sort(out2.begin(), out2.begin() + n);
  }) - copy_ms;
  expect(same_prefix(out, out2, n), "sort");
  std::printf("%-34s user %8.3f ms (merge sort, %.2f Gkeys/s)   library %8.3f ms (radix sort, %.2f Gkeys/s)\n", "sort", tu,
              n / tu / 1e6, tl, n / tl / 1e6);
  // the callers around the path (one reduction or one element-wise pass each); `out2` holds x sorted
  {
    auto single = [&](const char* what, double ms, double bytes) {
      std::printf("%-34s      %8.3f ms %5.1f%%\n", what, ms, bytes / ms / 1e6 / 80.0);
    };
    size_t at = 0;
    double t = best_ms([&] { at = thrust::min_element(x.begin(), x.end()) - x.begin(); });
    const unsigned smallest = x[at];
    expect(smallest == (unsigned)out2[0], "min_element");
    single("min_element", t, 4.0 * n);
    t = best_ms([&] { at = thrust::max_element(x.begin(), x.end(), my_less()) - x.begin(); });
    expect((unsigned)x[at] == (unsigned)out2[n - 1], "max_element");
    single("max_element, user comparator", t, 4.0 * n);
    const my_below never = {0u};
    t = best_ms([&] { at = thrust::find_if(x.begin(), x.end(), never) - x.begin(); });
    expect(at == n, "find_if of an absent element");
    single("find_if, nothing found", t, 4.0 * n);
    bool sorted = false;
    t = best_ms([&] { sorted = thrust::is_sorted(out2.begin(), out2.begin() + n); });
    expect(sorted, "is_sorted");
    single("is_sorted", t, 4.0 * n);  // every element is read once (twice by address, once from memory)
    const modulo by_thousand = {1000u};
    t = best_ms([&] { thrust::transform(x.begin(), x.end(), out.begin(), by_thousand); });
    expect((unsigned)out[n / 3] == (unsigned)x[n / 3] % 1000u && (unsigned)out[n - 1] == (unsigned)x[n - 1] % 1000u, "transform");
    single("transform, one input", t, 8.0 * n);
    t = best_ms([&] { thrust::transform(x.begin(), x.end(), vals.begin(), out.begin(), my_plus()); });
    expect((unsigned)out[n / 3] == (unsigned)x[n / 3] + (unsigned)vals[n / 3], "transform of two inputs");
    single("transform, two inputs", t, 12.0 * n);
    t = best_ms([&] { thrust::adjacent_difference(x.begin(), x.end(), out.begin()); });
    single("adjacent_difference", t, 8.0 * n);
    // every element of x looked up in the sorted copy of x: it is found, at a position that holds it
    t = best_ms([&] { thrust::lower_bound(out2.begin(), out2.begin() + n, x.begin(), x.end(), vout.begin()); });
    const unsigned probe = x[n / 3], where = vout[n / 3];
    expect((unsigned)out2[where] == probe && (where == 0 || (unsigned)out2[where - 1] < probe), "lower_bound");
    single("lower_bound, n values in n sorted", t, 8.0 * n);
  }
  std::printf("%d mismatches\n", g_failed);
  std::printf(g_failed ? "FAILED\n" : "PASSED\n");
  return g_failed ? 1 : 0;
}
