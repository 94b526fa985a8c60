// thrust::transform_reduce.
//
// transform_reduce(first, last, unary_op, init, binary_op) folds unary_op(x) over the range,
// starting from init; the result and every intermediate have the type of init
// (thrust/system/detail/generic/transform_reduce.inl:30-48).  On the device system
// unary_op is one of thrust::identity / negate / square and binary_op one of plus /
// minimum / maximum; the input is read once and nothing is staged.
#pragma once
#include <thrust/functional.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/reduce.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>

namespace thrust {

template <typename D, typename It, typename Fn, typename T, typename Op>
T transform_reduce(const detail::execution_policy_base<D>& exec, It first, It last, Fn unary_op, T init, Op binary_op);

namespace system {
namespace cpp {
template <typename D, typename It, typename Fn, typename T, typename Op>
T transform_reduce(execution_policy<D>&, It first, It last, Fn unary_op, T init, Op binary_op) {
  for (; first != last; ++first) init = binary_op(init, static_cast<T>(unary_op(*first)));
  return init;
}
}  // namespace cpp

namespace hip {
namespace detail {
// identity / negate / square on elements of init's type: applied inside the reduce kernel
template <typename D, typename It, typename Fn, typename T, typename Op>
T transform_reduce(execution_policy<D>& exec, It first, It last, Fn, T init, Op, std::true_type) {
  static_assert(binop_code<Op, T>::value >= 0,
                "thrust::transform_reduce on the device system supports thrust::plus, thrust::minimum and thrust::maximum");
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  device_input<It> source(stream, temp_source_of(exec), first, n);
  const void* in = n ? (const void*)source.ptr() : nullptr;
  temp_storage temp(stream, temp_source_of(exec));
  void* d_out = nullptr;
  std::size_t need = 0;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_transform_reduce(t, b, in, n, dtype_of<T>::value, unary_code<Fn, T>::value,
                                       binop_code<Op, T>::value, &init, d_out, stream);
  };
  throw_on_error(call(nullptr, &need), "transform_reduce: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_out = static_cast<char*>(temp.ptr()) + aligned;
  std::size_t bytes = aligned;
  throw_on_error(call(temp.ptr(), &bytes), "transform_reduce failed");
  return read_scalar<T>(d_out, stream, "transform_reduce: result copy");
}
// any other unary function: reduce over a transform iterator (needs a hipcc translation unit)
template <typename D, typename It, typename Fn, typename T, typename Op>
T transform_reduce(execution_policy<D>& exec, It first, It last, Fn fn, T init, Op op, std::false_type) {
  return thrust::reduce(exec, thrust::make_transform_iterator(first, fn), thrust::make_transform_iterator(last, fn),
                        init, op);
}
template <typename Fn, typename V, typename T, bool = is_abi_type<T>::value && std::is_same<V, T>::value>
struct transforms_in_kernel : std::integral_constant<bool, (unary_code<Fn, T>::value >= 0)> {};
template <typename Fn, typename V, typename T>
struct transforms_in_kernel<Fn, V, T, false> : std::false_type {};
}  // namespace detail

template <typename D, typename It, typename Fn, typename T, typename Op>
T transform_reduce(execution_policy<D>& exec, It first, It last, Fn fn, T init, Op op) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  static_assert(detail::is_device_input<It>::value,
                "thrust::transform_reduce on the device system needs device_ptr / device_vector iterators, raw device "
                "pointers or fancy iterators over them");
  return detail::transform_reduce(exec, first, last, fn, init, op, detail::transforms_in_kernel<Fn, V, T>());
}
}  // namespace hip
}  // namespace system

template <typename D, typename It, typename Fn, typename T, typename Op>
T transform_reduce(const detail::execution_policy_base<D>& exec, It first, It last, Fn unary_op, T init, Op binary_op) {
  return transform_reduce(detail::derived_cast(detail::strip_const(exec)), first, last, unary_op, init, binary_op);
}
template <typename It, typename Fn, typename T, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
T transform_reduce(It first, It last, Fn unary_op, T init, Op binary_op) {
  return thrust::transform_reduce(detail::policy_for<It>(), first, last, unary_op, init, binary_op);
}

}  // namespace thrust
