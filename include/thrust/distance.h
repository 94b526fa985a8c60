// thrust::distance (thrust/distance.h of the reference): last - first for the random-access
// iterators of this front end, std::distance for anything else.
#pragma once
#include <iterator>

#include <thrust/iterator/iterator_traits.h>

namespace thrust {
template <typename It>
inline typename thrust::iterator_difference<It>::type distance(It first, It last) {
  return std::distance(first, last);
}
}  // namespace thrust
