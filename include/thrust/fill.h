// thrust::fill / thrust::fill_n.
#pragma once
#include <algorithm>

#include <thrust/iterator/constant_iterator.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/transform.h>

namespace thrust {
namespace system {
namespace cpp {
template <typename D, typename It, typename T>
void fill(execution_policy<D>&, It first, It last, const T& value) { std::fill(first, last, value); }
}  // namespace cpp
namespace hip {
namespace detail {
template <typename V>
struct hands_on {
  __host__ __device__ V operator()(const V& x) const { return x; }
};
}  // namespace detail
// Into anything else a kernel can write through (a permutation, a zip, a strided view): the
// value as a constant range, copied element by element.
template <typename D, typename It, typename T>
typename std::enable_if<!(std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value)>::type fill(
    execution_policy<D>& exec, It first, It last, const T& value) {
  typedef typename iterator_value<It>::type V;
  thrust::constant_iterator<V> from(static_cast<V>(value));
  thrust::transform(exec, from, from + (last - first), first, detail::hands_on<V>());
}
template <typename D, typename It, typename T>
typename std::enable_if<std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value>::type fill(
    execution_policy<D>& exec, It first, It last, const T& value) {
  typedef typename iterator_value<It>::type V;
  static_assert(detail::is_abi_item<V>::value, "thrust::fill on the device system: items of 1, 2, 4 or 8 bytes");
  void* stream = detail::stream_of(exec);
  const V v = static_cast<V>(value);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return;
  detail::throw_on_error(thrust_amd_fill(thrust::detail::raw(first), n, sizeof(V), &v, stream), "fill failed");
  detail::synchronize(stream, "fill: synchronize");
}
}  // namespace hip
}  // namespace system

template <typename D, typename It, typename T>
void fill(const detail::execution_policy_base<D>& exec, It first, It last, const T& value) {
  fill(detail::derived_cast(detail::strip_const(exec)), first, last, value);
}
template <typename It, typename T>
void fill(It first, It last, const T& value) {
  thrust::fill(detail::policy_for<It>(), first, last, value);
}
template <typename D, typename It, typename Size, typename T>
It fill_n(const detail::execution_policy_base<D>& exec, It first, Size n, const T& value) {
  thrust::fill(exec, first, first + n, value);
  return first + n;
}
template <typename It, typename Size, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It fill_n(It first, Size n, const T& value) {
  thrust::fill(first, first + n, value);
  return first + n;
}
}  // namespace thrust
