// thrust::generate, generate_n: every element becomes gen()
// (thrust/system/detail/generic/generate.inl:33-77: a for_each that assigns; testing/generate.cu).
// On the device system every thread calls its own copy of the generator.
#pragma once
#include <cstddef>

#include <thrust/transform.h>

namespace thrust {
namespace detail {
template <typename Gen>
struct assigns_generated {
  mutable Gen gen;
  template <typename V>
  __host__ __device__ void operator()(V& x) const { x = gen(); }
};
}  // namespace detail

template <typename D, typename It, typename Gen>
void generate(const detail::execution_policy_base<D>& exec, It first, It last, Gen gen) {
  const detail::assigns_generated<Gen> f = {gen};
  thrust::for_each(exec, first, last, f);
}
template <typename D, typename It, typename Size, typename Gen>
It generate_n(const detail::execution_policy_base<D>& exec, It first, Size n, Gen gen) {
  thrust::generate(exec, first, first + (std::ptrdiff_t)n, gen);
  return first + (std::ptrdiff_t)n;
}
template <typename It, typename Gen, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void generate(It first, It last, Gen gen) {
  thrust::generate(detail::policy_for<It>(), first, last, gen);
}
template <typename It, typename Size, typename Gen,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It generate_n(It first, Size n, Gen gen) {
  return thrust::generate_n(detail::policy_for<It>(), first, n, gen);
}

}  // namespace thrust
