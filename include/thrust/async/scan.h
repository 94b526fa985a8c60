// thrust::async::inclusive_scan and thrust::async::exclusive_scan.
//
// Enqueue the scan and return a device_event (thrust/async/scan.h of the reference; device
// path thrust/system/cuda/detail/async/inclusive_scan.h, exclusive_scan.h).  The operator is
// thrust::plus (default), minimum or maximum; output may be the input range.
#pragma once
#include <thrust/functional.h>
#include <thrust/future.h>

namespace thrust {
namespace async {

namespace detail {
template <typename In, typename Out, typename T, typename Op>
struct scan_checks {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  static_assert((std::is_pointer<In>::value || thrust::detail::is_device_iterator<In>::value) &&
                    (std::is_pointer<Out>::value || thrust::detail::is_device_iterator<Out>::value),
                "asynchronous scans need device_ptr / device_vector iterators or raw device pointers");
  static_assert(thrust::system::hip::detail::is_abi_type<V>::value && std::is_same<V, T>::value &&
                    std::is_same<typename iterator_value<Out>::type, V>::value,
                "asynchronous scans: input, output and init must share one arithmetic type");
  static_assert(thrust::system::hip::detail::binop_code<Op, V>::value >= 0,
                "asynchronous scans support thrust::plus, thrust::minimum and thrust::maximum");
};
}  // namespace detail

template <typename D, typename In, typename Out, typename Op>
device_event inclusive_scan(const thrust::detail::execution_policy_base<D>& exec, In first, In last, Out result, Op) {
  namespace backend = thrust::system::hip::detail;
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  (void)sizeof(detail::scan_checks<In, Out, V, Op>);
  auto& pol = thrust::detail::derived_cast(thrust::detail::strip_const(exec));
  backend::async_context ctx = backend::context_of(pol, 0);
  const uint64_t n = (uint64_t)(last - first);
  if (n) {
    std::shared_ptr<backend::temp_storage> temp = backend::async_temp(ctx, backend::temp_source_of(pol));
    void* stream = ctx.stream();
    backend::run(*temp, 0, "async inclusive_scan failed", [&](void* t, std::size_t* b) {
      return thrust_amd_inclusive_scan(t, b, thrust::detail::raw(first), thrust::detail::raw(result), n,
                                       backend::dtype_of<V>::value, backend::binop_code<Op, V>::value, stream);
    });
  }
  return device_event(ctx.keep);
}
template <typename D, typename In, typename Out>
device_event inclusive_scan(const thrust::detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  return thrust::async::inclusive_scan(exec, first, last, result, thrust::plus<>());
}
template <typename In, typename Out, typename Op,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<In>::value>::type>
device_event inclusive_scan(In first, In last, Out result, Op op) {
  return thrust::async::inclusive_scan(thrust::device, first, last, result, op);
}
template <typename In, typename Out>
device_event inclusive_scan(In first, In last, Out result) {
  return thrust::async::inclusive_scan(thrust::device, first, last, result, thrust::plus<>());
}

template <typename D, typename In, typename Out, typename T, typename Op>
device_event exclusive_scan(const thrust::detail::execution_policy_base<D>& exec, In first, In last, Out result, T init,
                            Op) {
  namespace backend = thrust::system::hip::detail;
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  (void)sizeof(detail::scan_checks<In, Out, T, Op>);
  auto& pol = thrust::detail::derived_cast(thrust::detail::strip_const(exec));
  backend::async_context ctx = backend::context_of(pol, 0);
  const uint64_t n = (uint64_t)(last - first);
  if (n) {
    std::shared_ptr<backend::temp_storage> temp = backend::async_temp(ctx, backend::temp_source_of(pol));
    void* stream = ctx.stream();
    backend::run(*temp, 0, "async exclusive_scan failed", [&](void* t, std::size_t* b) {
      return thrust_amd_exclusive_scan(t, b, thrust::detail::raw(first), thrust::detail::raw(result), n,
                                       backend::dtype_of<V>::value, backend::binop_code<Op, V>::value, &init, stream);
    });
  }
  return device_event(ctx.keep);
}
template <typename D, typename In, typename Out, typename T>
device_event exclusive_scan(const thrust::detail::execution_policy_base<D>& exec, In first, In last, Out result, T init) {
  return thrust::async::exclusive_scan(exec, first, last, result, init, thrust::plus<>());
}
template <typename In, typename Out, typename T, typename Op,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<In>::value>::type>
device_event exclusive_scan(In first, In last, Out result, T init, Op op) {
  return thrust::async::exclusive_scan(thrust::device, first, last, result, init, op);
}
template <typename In, typename Out, typename T,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<In>::value>::type>
device_event exclusive_scan(In first, In last, Out result, T init) {
  return thrust::async::exclusive_scan(thrust::device, first, last, result, init, thrust::plus<>());
}

}  // namespace async
}  // namespace thrust
