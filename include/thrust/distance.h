// thrust::distance: how many increments lead from first to last (thrust/distance.h:60;
// testing/distance.cu).  A subtraction for the random-access ranges every algorithm here
// takes, a walk for the rest.
#pragma once
#include <iterator>

#include <thrust/iterator/iterator_traits.h>

namespace thrust {
namespace detail {
template <typename It>
inline __host__ __device__ auto distance_of(It first, It last, int) -> decltype(last - first) { return last - first; }
template <typename It>
inline typename std::iterator_traits<It>::difference_type distance_of(It first, It last, long) {
  return std::distance(first, last);
}
}  // namespace detail
template <typename It>
inline __host__ __device__ typename thrust::iterator_difference<It>::type distance(It first, It last) {
  return detail::distance_of(first, last, 0);
}
}  // namespace thrust
