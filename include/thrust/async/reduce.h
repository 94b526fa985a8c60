// thrust::async::reduce and thrust::async::reduce_into.
//
// reduce(policy, first, last, init, op) enqueues the reduction and returns a device_future
// holding the value; reduce_into(..., output, init, op) writes the value to *output (device
// memory) and returns a device_event (thrust/async/reduce.h:62-434 of the reference;
// device path thrust/system/cuda/detail/async/reduce.h).  Defaults as for thrust::reduce:
// init = value_type(0), op = plus.  See thrust/future.h for streams and dependencies.
#pragma once
#include <thrust/functional.h>
#include <thrust/future.h>

namespace thrust {
namespace async {

namespace detail {
// Enqueues the reduction on the context's stream; d_result == nullptr: a slot is taken
// from the temporary storage.  Returns the device address of the value.
template <typename P, typename It, typename T, typename Op>
inline const T* enqueue_reduce(P& pol, system::hip::detail::async_context& ctx, It first, It last, T init, Op, T* d_result) {
  namespace backend = thrust::system::hip::detail;
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  static_assert(std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value,
                "thrust::async::reduce needs device_ptr / device_vector iterators or raw device pointers");
  static_assert(backend::is_abi_type<T>::value && std::is_same<V, T>::value,
                "thrust::async::reduce: init must have the (arithmetic) element type");
  static_assert(backend::binop_code<Op, T>::value >= 0,
                "thrust::async::reduce supports thrust::plus, thrust::minimum and thrust::maximum");
  void* stream = ctx.stream();
  const uint64_t n = (uint64_t)(last - first);
  const void* in = n ? (const void*)thrust::detail::raw(first) : nullptr;
  std::shared_ptr<backend::temp_storage> temp = backend::async_temp(ctx, backend::temp_source_of(pol));
  std::size_t need = 0;
  backend::throw_on_error(thrust_amd_reduce(nullptr, &need, in, n, backend::dtype_of<T>::value,
                                            backend::binop_code<Op, T>::value, &init, nullptr, stream),
                          "async reduce: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp->ensure(aligned + 256);
  T* d_out = d_result ? d_result : reinterpret_cast<T*>(static_cast<char*>(temp->ptr()) + aligned);
  std::size_t bytes = aligned;
  backend::throw_on_error(thrust_amd_reduce(temp->ptr(), &bytes, in, n, backend::dtype_of<T>::value,
                                            backend::binop_code<Op, T>::value, &init, d_out, stream),
                          "async reduce failed");
  return d_out;
}
}  // namespace detail

template <typename D, typename It, typename T, typename Op>
device_future<T> reduce(const thrust::detail::execution_policy_base<D>& exec, It first, It last, T init, Op op) {
  auto& pol = thrust::detail::derived_cast(thrust::detail::strip_const(exec));
  system::hip::detail::async_context ctx = system::hip::detail::context_of(pol, 0);
  const T* d_value = detail::enqueue_reduce(pol, ctx, first, last, init, op, (T*)nullptr);
  return device_future<T>(ctx.keep, d_value);
}
template <typename D, typename It, typename T>
device_future<T> reduce(const thrust::detail::execution_policy_base<D>& exec, It first, It last, T init) {
  return thrust::async::reduce(exec, first, last, init, thrust::plus<T>());
}
template <typename D, typename It>
device_future<typename std::remove_const<typename iterator_value<It>::type>::type> reduce(
    const thrust::detail::execution_policy_base<D>& exec, It first, It last) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type T;
  return thrust::async::reduce(exec, first, last, T(0), thrust::plus<T>());
}
template <typename It, typename T, typename Op,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<It>::value>::type>
device_future<T> reduce(It first, It last, T init, Op op) {
  return thrust::async::reduce(thrust::device, first, last, init, op);
}
template <typename It, typename T,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<It>::value>::type>
device_future<T> reduce(It first, It last, T init) {
  return thrust::async::reduce(thrust::device, first, last, init, thrust::plus<T>());
}
template <typename It>
device_future<typename std::remove_const<typename iterator_value<It>::type>::type> reduce(It first, It last) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type T;
  return thrust::async::reduce(thrust::device, first, last, T(0), thrust::plus<T>());
}

template <typename D, typename It, typename Out, typename T, typename Op>
device_event reduce_into(const thrust::detail::execution_policy_base<D>& exec, It first, It last, Out output, T init, Op op) {
  static_assert(std::is_same<typename iterator_value<Out>::type, T>::value,
                "thrust::async::reduce_into: the output element type must be the type of init");
  auto& pol = thrust::detail::derived_cast(thrust::detail::strip_const(exec));
  system::hip::detail::async_context ctx = system::hip::detail::context_of(pol, 0);
  (void)detail::enqueue_reduce(pol, ctx, first, last, init, op, thrust::detail::raw(output));
  return device_event(ctx.keep);
}
template <typename D, typename It, typename Out, typename T>
device_event reduce_into(const thrust::detail::execution_policy_base<D>& exec, It first, It last, Out output, T init) {
  return thrust::async::reduce_into(exec, first, last, output, init, thrust::plus<T>());
}
template <typename D, typename It, typename Out>
device_event reduce_into(const thrust::detail::execution_policy_base<D>& exec, It first, It last, Out output) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type T;
  return thrust::async::reduce_into(exec, first, last, output, T(0), thrust::plus<T>());
}
template <typename It, typename Out, typename T, typename Op,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<It>::value>::type>
device_event reduce_into(It first, It last, Out output, T init, Op op) {
  return thrust::async::reduce_into(thrust::device, first, last, output, init, op);
}
template <typename It, typename Out, typename T,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<It>::value>::type>
device_event reduce_into(It first, It last, Out output, T init) {
  return thrust::async::reduce_into(thrust::device, first, last, output, init, thrust::plus<T>());
}
template <typename It, typename Out,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<It>::value>::type>
device_event reduce_into(It first, It last, Out output) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type T;
  return thrust::async::reduce_into(thrust::device, first, last, output, T(0), thrust::plus<T>());
}

}  // namespace async
}  // namespace thrust
