// thrust::async::sort and thrust::async::stable_sort.
//
// Enqueue the (stable) radix sort of the range and return a device_event
// (thrust/async/sort.h:60-270 of the reference).  The comparison is thrust::less (default)
// or thrust::greater on an arithmetic key type.
#pragma once
#include <thrust/functional.h>
#include <thrust/future.h>

namespace thrust {
namespace async {

template <typename D, typename It, typename Comp>
device_event stable_sort(const thrust::detail::execution_policy_base<D>& exec, It first, It last, Comp) {
  namespace backend = thrust::system::hip::detail;
  typedef typename std::remove_const<typename iterator_value<It>::type>::type K;
  static_assert(std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value,
                "thrust::async::sort needs device_ptr / device_vector iterators or raw device pointers");
  static_assert(backend::is_abi_type<K>::value, "thrust::async::sort needs an arithmetic key type");
  static_assert(backend::order_code<Comp, K>::value >= 0, "thrust::async::sort supports thrust::less and thrust::greater");
  auto& pol = thrust::detail::derived_cast(thrust::detail::strip_const(exec));
  backend::async_context ctx = backend::context_of(pol, 0);
  const uint64_t n = (uint64_t)(last - first);
  if (n > 1) {
    std::shared_ptr<backend::temp_storage> temp = backend::async_temp(ctx, backend::temp_source_of(pol));
    void* stream = ctx.stream();
    backend::run(*temp, 0, "async sort failed", [&](void* t, std::size_t* b) {
      return thrust_amd_sort_keys(t, b, thrust::detail::raw(first), n, backend::dtype_of<K>::value,
                                  backend::order_code<Comp, K>::value, 0, (int)(8 * sizeof(K)), stream);
    });
  }
  return device_event(ctx.keep);
}
template <typename D, typename It>
device_event stable_sort(const thrust::detail::execution_policy_base<D>& exec, It first, It last) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type K;
  return thrust::async::stable_sort(exec, first, last, thrust::less<K>());
}
template <typename It, typename Comp,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<It>::value>::type>
device_event stable_sort(It first, It last, Comp comp) {
  return thrust::async::stable_sort(thrust::device, first, last, comp);
}
template <typename It>
device_event stable_sort(It first, It last) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type K;
  return thrust::async::stable_sort(thrust::device, first, last, thrust::less<K>());
}

// the radix sort is stable, so sort is the same call
template <typename D, typename It, typename Comp>
device_event sort(const thrust::detail::execution_policy_base<D>& exec, It first, It last, Comp comp) {
  return thrust::async::stable_sort(exec, first, last, comp);
}
template <typename D, typename It>
device_event sort(const thrust::detail::execution_policy_base<D>& exec, It first, It last) {
  return thrust::async::stable_sort(exec, first, last);
}
template <typename It, typename Comp,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<It>::value>::type>
device_event sort(It first, It last, Comp comp) {
  return thrust::async::stable_sort(thrust::device, first, last, comp);
}
template <typename It>
device_event sort(It first, It last) {
  return thrust::async::stable_sort(first, last);
}

}  // namespace async
}  // namespace thrust
