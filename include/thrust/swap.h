// thrust::swap_ranges: exchanges two ranges element by element, returns the end of the second
// (thrust/system/detail/generic/swap_ranges.inl:35-70: a for_each over the zipped ranges;
// testing/swap_ranges.cu).
#pragma once
#include <cstddef>

#include <thrust/iterator/zip_iterator.h>
#include <thrust/transform.h>
#include <thrust/tuple.h>

namespace thrust {
namespace detail {
struct swaps_pair {
  template <typename Tuple>
  __host__ __device__ void operator()(Tuple t) const {
    const auto first_value = thrust::get<0>(t);  // a copy: get<> yields a reference
    thrust::get<0>(t) = thrust::get<1>(t);
    thrust::get<1>(t) = first_value;
  }
};
}  // namespace detail

template <typename D, typename It1, typename It2>
It2 swap_ranges(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2) {
  const std::ptrdiff_t n = last1 - first1;
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first1, first2));
  thrust::for_each(exec, zipped, zipped + n, detail::swaps_pair());
  return first2 + n;
}
template <typename It1, typename It2, typename = typename std::enable_if<!detail::is_execution_policy<It1>::value>::type>
It2 swap_ranges(It1 first1, It1 last1, It2 first2) {
  return thrust::swap_ranges(detail::policy_for<It1>(), first1, last1, first2);
}

}  // namespace thrust
