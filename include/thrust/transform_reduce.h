// thrust::transform_reduce.
//
// transform_reduce(first, last, unary_op, init, binary_op) folds unary_op(x) over the range,
// starting from init; the result and every intermediate have the type of init
// (thrust/system/detail/generic/transform_reduce.inl:30-48).  On the device system
// unary_op is one of thrust::identity / negate / square and binary_op one of plus /
// minimum / maximum; the input is read once and nothing is staged.
#pragma once
#include <thrust/functional.h>
#include <thrust/system/hip/detail/backend.h>

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
template <typename D, typename It, typename Fn, typename T, typename Op>
T transform_reduce(execution_policy<D>& exec, It first, It last, Fn, T init, Op) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  static_assert(std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value,
                "thrust::transform_reduce on the device system needs device_ptr / device_vector iterators or raw device pointers");
  static_assert(detail::is_abi_type<T>::value && std::is_same<V, T>::value,
                "thrust::transform_reduce on the device system: init must have the (arithmetic) element type");
  static_assert(detail::unary_code<Fn, T>::value >= 0,
                "thrust::transform_reduce on the device system supports thrust::identity, thrust::negate and thrust::square");
  static_assert(detail::binop_code<Op, T>::value >= 0,
                "thrust::transform_reduce on the device system supports thrust::plus, thrust::minimum and thrust::maximum");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  const void* in = n ? (const void*)thrust::detail::raw(first) : nullptr;
  detail::temp_storage temp(stream, detail::temp_source_of(exec));
  void* d_out = nullptr;
  std::size_t need = 0;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_transform_reduce(t, b, in, n, detail::dtype_of<T>::value, detail::unary_code<Fn, T>::value,
                                       detail::binop_code<Op, T>::value, &init, d_out, stream);
  };
  detail::throw_on_error(call(nullptr, &need), "transform_reduce: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_out = static_cast<char*>(temp.ptr()) + aligned;
  std::size_t bytes = aligned;
  detail::throw_on_error(call(temp.ptr(), &bytes), "transform_reduce failed");
  return detail::read_scalar<T>(d_out, stream, "transform_reduce: result copy");
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
