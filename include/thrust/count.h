// thrust::count and thrust::count_if.
//
// count(first, last, value) counts elements equal to value; count_if counts elements
// for which the predicate holds.  The result type is the iterator's difference type
// (thrust/system/detail/generic/count.inl:45-74: a transform_reduce of 0/1 with plus).
// On the device system the predicate must be a comparison of the element with a
// constant (`_1 < t`, thrust::identity, thrust::logical_not).
#pragma once
#include <cstddef>

#include <thrust/functional.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/reduce.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>

namespace thrust {

template <typename D, typename It, typename Pred>
std::ptrdiff_t count_if(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred);
template <typename D, typename It, typename T>
std::ptrdiff_t count(const detail::execution_policy_base<D>& exec, It first, It last, const T& value);

namespace system {
namespace detail {
namespace generic {
// count(value) = count_if(x == value), compared in the element type
template <typename D, typename It, typename T>
std::ptrdiff_t count(thrust::execution_policy<D>& exec, It first, It last, const T& value) {
  using namespace thrust::placeholders;
  return thrust::count_if(exec, first, last, _1 == value);
}
}  // namespace generic
}  // namespace detail

namespace cpp {
template <typename D, typename It, typename Pred>
std::ptrdiff_t count_if(execution_policy<D>&, It first, It last, Pred pred) {
  std::ptrdiff_t c = 0;
  for (; first != last; ++first) c += pred(*first) ? 1 : 0;
  return c;
}
}  // namespace cpp

namespace hip {
namespace detail {
template <typename Pred>
struct counts_one {  // a user predicate as a 0 / 1 summand
  mutable Pred pred;  // a caller's predicate need not be const-callable
  template <typename V>
  __host__ __device__ long long operator()(const V& x) const { return pred(x) ? 1 : 0; }
};

// recognised predicate on arithmetic elements: the comparison is done inside the reduce kernel
template <typename D, typename It, typename Pred>
std::ptrdiff_t count_if(execution_policy<D>& exec, It first, It last, Pred pred, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return 0;
  const V threshold = unary_pred<Pred, V>::threshold(pred);
  const int cmp = unary_pred<Pred, V>::cmp(pred);
  device_input<It> source(stream, temp_source_of(exec), first, n);
  temp_storage temp(stream, temp_source_of(exec));
  uint64_t* d_count = nullptr;
  std::size_t need = 0;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_count_if(t, b, source.ptr(), n, dtype_of<V>::value, cmp, &threshold, d_count, stream);
  };
  throw_on_error(call(nullptr, &need), "count_if: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_count = reinterpret_cast<uint64_t*>(static_cast<char*>(temp.ptr()) + aligned);
  std::size_t bytes = aligned;
  throw_on_error(call(temp.ptr(), &bytes), "count_if failed");
  return (std::ptrdiff_t)read_scalar<uint64_t>(d_count, stream, "count_if: result copy");
}
// any other predicate: a sum over a transform iterator (needs a hipcc translation unit)
template <typename D, typename It, typename Pred>
std::ptrdiff_t count_if(execution_policy<D>& exec, It first, It last, Pred pred, std::false_type) {
  const counts_one<Pred> one = {pred};
  return (std::ptrdiff_t)thrust::reduce(exec, thrust::make_transform_iterator(first, one),
                                        thrust::make_transform_iterator(last, one), (long long)0,
                                        thrust::plus<long long>());
}
template <typename Pred, typename V, bool = is_abi_type<V>::value>
struct count_in_kernel : std::integral_constant<bool, unary_pred<Pred, V>::supported> {};
template <typename Pred, typename V>
struct count_in_kernel<Pred, V, false> : std::false_type {};
}  // namespace detail

template <typename D, typename It, typename Pred>
std::ptrdiff_t count_if(execution_policy<D>& exec, It first, It last, Pred pred) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  static_assert(detail::is_device_input<It>::value,
                "thrust::count_if on the device system needs device_ptr / device_vector iterators, raw device pointers "
                "or fancy iterators over them");
  return detail::count_if(exec, first, last, pred, detail::count_in_kernel<Pred, V>());
}
}  // namespace hip
}  // namespace system

template <typename D, typename It, typename Pred>
std::ptrdiff_t count_if(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return count_if(detail::derived_cast(detail::strip_const(exec)), first, last, pred);
}
template <typename D, typename It, typename T>
std::ptrdiff_t count(const detail::execution_policy_base<D>& exec, It first, It last, const T& value) {
  using thrust::system::detail::generic::count;
  return count(detail::derived_cast(detail::strip_const(exec)), first, last, value);
}
template <typename It, typename Pred>
std::ptrdiff_t count_if(It first, It last, Pred pred) {
  return thrust::count_if(detail::policy_for<It>(), first, last, pred);
}
template <typename It, typename T>
std::ptrdiff_t count(It first, It last, const T& value) {
  return thrust::count(detail::policy_for<It>(), first, last, value);
}

}  // namespace thrust
