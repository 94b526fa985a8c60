// thrust::reverse (in place) and thrust::reverse_copy
// (thrust/system/detail/generic/reverse.inl:33-72; testing/reverse.cu).  reverse_copy is a gather
// through the mirrored positions; reverse mirrors a copy of the range back onto it.
#pragma once
#include <algorithm>
#include <cstddef>

#include <thrust/device_vector.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/transform.h>

namespace thrust {

template <typename D, typename In, typename Out>
Out reverse_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result);

namespace detail {
struct mirrored_position {
  std::ptrdiff_t last_index;
  __host__ __device__ std::ptrdiff_t operator()(std::ptrdiff_t i) const { return last_index - i; }
};
}  // namespace detail

namespace system {
namespace cpp {
template <typename D, typename It>
void reverse(execution_policy<D>&, It first, It last) {
  std::reverse(first, last);
}
template <typename D, typename In, typename Out>
Out reverse_copy(execution_policy<D>&, In first, In last, Out result) {
  while (first != last) *result++ = *--last;
  return result;
}
}  // namespace cpp
namespace hip {
template <typename D, typename In, typename Out>
Out reverse_copy(execution_policy<D>& exec, In first, In last, Out result) {
  const std::ptrdiff_t n = last - first;
  if (n == 0) return result;
  const thrust::detail::mirrored_position mirror = {n - 1};
  thrust::counting_iterator<std::ptrdiff_t> zero(0);
  return thrust::gather(exec, thrust::make_transform_iterator(zero, mirror), thrust::make_transform_iterator(zero + n, mirror),
                        first, result);
}
template <typename D, typename It>
void reverse(execution_policy<D>& exec, It first, It last) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  if (last - first < 2) return;
  thrust::device_vector<V> input(first, last);
  thrust::reverse_copy(exec, input.begin(), input.end(), first);
}
}  // namespace hip
}  // namespace system

template <typename D, typename In, typename Out>
Out reverse_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  return reverse_copy(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
template <typename D, typename It>
void reverse(const detail::execution_policy_base<D>& exec, It first, It last) {
  reverse(detail::derived_cast(detail::strip_const(exec)), first, last);
}
template <typename In, typename Out, typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out reverse_copy(In first, In last, Out result) {
  return thrust::reverse_copy(detail::policy_for<Out>(), first, last, result);
}
template <typename It>
void reverse(It first, It last) {
  thrust::reverse(detail::policy_for<It>(), first, last);
}

}  // namespace thrust
