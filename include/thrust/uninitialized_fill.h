// thrust::uninitialized_fill, uninitialized_fill_n: for the trivially copyable element types of
// the device system, constructing a copy is assigning it
// (thrust/system/detail/generic/uninitialized_fill.inl:33-118 takes the same route for types with a
// trivial copy constructor; testing/uninitialized_fill.cu).
#pragma once
#include <cstddef>

#include <thrust/fill.h>

namespace thrust {

template <typename D, typename It, typename T>
void uninitialized_fill(const detail::execution_policy_base<D>& exec, It first, It last, const T& value) {
  thrust::fill(exec, first, last, value);
}
template <typename D, typename It, typename Size, typename T>
It uninitialized_fill_n(const detail::execution_policy_base<D>& exec, It first, Size n, const T& value) {
  thrust::fill(exec, first, first + (std::ptrdiff_t)n, value);
  return first + (std::ptrdiff_t)n;
}
template <typename It, typename T, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void uninitialized_fill(It first, It last, const T& value) {
  thrust::fill(first, last, value);
}
template <typename It, typename Size, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It uninitialized_fill_n(It first, Size n, const T& value) {
  thrust::fill(first, first + (std::ptrdiff_t)n, value);
  return first + (std::ptrdiff_t)n;
}

}  // namespace thrust
