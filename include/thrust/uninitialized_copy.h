// thrust::uninitialized_copy, uninitialized_copy_n: for the trivially copyable element types of
// the device system, constructing a copy is copying the bytes
// (thrust/system/detail/generic/uninitialized_copy.inl:33-180 takes the same route for types with a
// trivial copy constructor; testing/uninitialized_copy.cu).
#pragma once
#include <cstddef>

#include <thrust/copy.h>

namespace thrust {

template <typename D, typename In, typename Out>
Out uninitialized_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  return thrust::copy(exec, first, last, result);
}
template <typename D, typename In, typename Size, typename Out>
Out uninitialized_copy_n(const detail::execution_policy_base<D>& exec, In first, Size n, Out result) {
  return thrust::copy(exec, first, first + (std::ptrdiff_t)n, result);
}
template <typename In, typename Out, typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out uninitialized_copy(In first, In last, Out result) {
  return thrust::copy(first, last, result);
}
template <typename In, typename Size, typename Out,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out uninitialized_copy_n(In first, Size n, Out result) {
  return thrust::copy(first, first + (std::ptrdiff_t)n, result);
}

}  // namespace thrust
