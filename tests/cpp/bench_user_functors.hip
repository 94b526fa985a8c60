// Timing of the paths that run in kernels instantiated in the user's translation unit:
// user-defined operators, predicates and comparators through the thrust:: front end.
// Every line is the blocking call as a user makes it (temporary storage from the caching
// arena, result sizes copied back), best of five after one warm-up, inputs resident in HBM.
// Bytes are the algorithmic ones of the library path for the same job (a range read once,
// a result written once), so the percentages compare with the tuned kernels' figures.
//
//   tests/cpp/bin/bench_user_functors [log2 of the element count, default 27]
#include <thrust/device_vector.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/merge.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/set_operations.h>
#include <thrust/sort.h>
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
static void line(const char* what, double ms, double bytes) {
  std::printf("%-52s %9.3f ms %8.0f GB/s %5.1f%%\n", what, ms, bytes / ms / 1e6, bytes / ms / 1e6 / 80.0);
}

int main(int argc, char** argv) {
  const int lg = argc > 1 ? std::atoi(argv[1]) : 27;
  const size_t n = (size_t)1 << lg;
  std::printf("user functors through the front end, n = 2^%d uint32\n", lg);
  thrust::counting_iterator<uint64_t> index(0);
  thrust::device_vector<unsigned> x(n), y(n), out(2 * n), vals(n, 1u), vout(n);
  thrust::copy(thrust::make_transform_iterator(index, scramble{1}), thrust::make_transform_iterator(index, scramble{1}) + n,
               x.begin());
  volatile unsigned sink = 0;

  line("reduce, user plus", best_ms([&] { sink = thrust::reduce(x.begin(), x.end(), 0u, my_plus()); }), 4.0 * n);
  line("reduce, transform_iterator, thrust::plus",
       best_ms([&] {
         sink = thrust::reduce(thrust::make_transform_iterator(x.begin(), modulo{1001}),
                               thrust::make_transform_iterator(x.begin(), modulo{1001}) + n, 0u);
       }),
       4.0 * n);
  line("inclusive_scan, user plus", best_ms([&] { thrust::inclusive_scan(x.begin(), x.end(), out.begin(), my_plus()); }),
       8.0 * n);

  // sorted keys with runs of about eight
  thrust::copy(thrust::make_transform_iterator(x.begin(), modulo{(unsigned)(n / 8)}),
               thrust::make_transform_iterator(x.begin(), modulo{(unsigned)(n / 8)}) + n, y.begin());
  thrust::sort(y.begin(), y.end());
  size_t runs = 0;
  line("unique_copy, user equality",
       best_ms([&] { runs = thrust::unique_copy(y.begin(), y.end(), out.begin(), my_equal()) - out.begin(); }),
       4.0 * n + 4.0 * (n / 8));
  line("reduce_by_key, user equality and plus",
       best_ms([&] {
         thrust::reduce_by_key(y.begin(), y.end(), vals.begin(), out.begin(), vout.begin(), my_equal(), my_plus());
       }),
       8.0 * n + 8.0 * (n / 8));
  std::printf("  (%zu runs)\n", runs);

  // two sorted ranges of n / 2 with duplicates in and across them
  const size_t m = n / 2;
  thrust::device_vector<unsigned> a(m), b(m);
  thrust::copy(thrust::make_transform_iterator(x.begin(), modulo{(unsigned)(m / 4)}),
               thrust::make_transform_iterator(x.begin(), modulo{(unsigned)(m / 4)}) + m, a.begin());
  thrust::copy(thrust::make_transform_iterator(x.begin() + m, modulo{(unsigned)(m / 2)}),
               thrust::make_transform_iterator(x.begin() + m, modulo{(unsigned)(m / 2)}) + m, b.begin());
  thrust::sort(a.begin(), a.end());
  thrust::sort(b.begin(), b.end());
  line("merge, user less", best_ms([&] { thrust::merge(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less()); }),
       8.0 * n);
  size_t kept = 0;
  const double union_ms = best_ms(
      [&] { kept = thrust::set_union(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less()) - out.begin(); });
  line("set_union, user less", union_ms, 4.0 * n + 4.0 * kept);
  const double inter_ms = best_ms([&] {
    kept = thrust::set_intersection(a.begin(), a.end(), b.begin(), b.end(), out.begin(), my_less()) - out.begin();
  });
  line("set_intersection, user less", inter_ms, 4.0 * n + 4.0 * kept);

  // the sort last: it is in place, every repetition sorts a fresh copy (the copy is timed separately)
  const double copy_ms = best_ms([&] { thrust::copy(x.begin(), x.end(), out.begin()); });
  const double sort_ms = best_ms([&] {
    thrust::copy(x.begin(), x.end(), out.begin());
    thrust::sort(out.begin(), out.begin() + n, my_less());
  });
  int passes = 0;
  for (size_t run = 4096; run < n; run <<= 1) ++passes;
  line("sort, user less (merge sort)", sort_ms - copy_ms, (1.0 + passes) * 8.0 * n);
  std::printf("  (%.2f Gkeys/s)\n", n / (sort_ms - copy_ms) / 1e6);
  (void)sink;
  return 0;
}
