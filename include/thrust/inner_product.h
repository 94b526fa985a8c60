// thrust::inner_product.
//
// inner_product(first1, last1, first2, init) = init + sum of a[i] * b[i]; the products
// and the sum are made in the type of init (multiplies<T> and plus<T>,
// thrust/system/detail/generic/inner_product.inl:33-65).  The four-functor overload is
// available on the host system; the device system supports plus / multiplies.
#pragma once
#include <thrust/functional.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>

namespace thrust {

template <typename D, typename It1, typename It2, typename T>
T inner_product(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2, T init);
template <typename D, typename It1, typename It2, typename T, typename Op1, typename Op2>
T inner_product(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2, T init, Op1 op1,
                Op2 op2);

namespace system {
namespace detail {
namespace generic {
template <typename D, typename It1, typename It2, typename T>
T inner_product(thrust::execution_policy<D>& exec, It1 first1, It1 last1, It2 first2, T init) {
  return thrust::inner_product(exec, first1, last1, first2, init, thrust::plus<T>(), thrust::multiplies<T>());
}
}  // namespace generic
}  // namespace detail

namespace cpp {
template <typename D, typename It1, typename It2, typename T, typename Op1, typename Op2>
T inner_product(execution_policy<D>&, It1 first1, It1 last1, It2 first2, T init, Op1 op1, Op2 op2) {
  for (; first1 != last1; ++first1, ++first2) init = op1(init, op2(*first1, *first2));
  return init;
}
}  // namespace cpp

namespace hip {
template <typename D, typename It1, typename It2, typename T, typename Op1, typename Op2>
T inner_product(execution_policy<D>& exec, It1 first1, It1 last1, It2 first2, T init, Op1, Op2) {
  typedef typename std::remove_const<typename iterator_value<It1>::type>::type V1;
  typedef typename std::remove_const<typename iterator_value<It2>::type>::type V2;
  static_assert(detail::is_device_input<It1>::value && detail::is_device_input<It2>::value,
                "thrust::inner_product on the device system needs device_ptr / device_vector iterators, raw device "
                "pointers or fancy iterators over them");
  static_assert(detail::is_abi_type<T>::value && std::is_same<V1, T>::value && std::is_same<V2, T>::value,
                "thrust::inner_product on the device system: both ranges and init must share one arithmetic type");
  static_assert(detail::binop_code<Op1, T>::value == THRUST_AMD_PLUS &&
                    (std::is_same<Op2, thrust::multiplies<T> >::value || std::is_same<Op2, thrust::multiplies<void> >::value),
                "thrust::inner_product on the device system supports thrust::plus with thrust::multiplies");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last1 - first1);
  if (n == 0) return init;
  detail::device_input<It1> source1(stream, detail::temp_source_of(exec), first1, n);
  detail::device_input<It2> source2(stream, detail::temp_source_of(exec), first2, n);
  detail::temp_storage temp(stream, detail::temp_source_of(exec));
  void* d_out = nullptr;
  std::size_t need = 0;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_inner_product(t, b, source1.ptr(), source2.ptr(), n,
                                    detail::dtype_of<T>::value, &init, d_out, stream);
  };
  detail::throw_on_error(call(nullptr, &need), "inner_product: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_out = static_cast<char*>(temp.ptr()) + aligned;
  std::size_t bytes = aligned;
  detail::throw_on_error(call(temp.ptr(), &bytes), "inner_product failed");
  return detail::read_scalar<T>(d_out, stream, "inner_product: result copy");
}
}  // namespace hip
}  // namespace system

template <typename D, typename It1, typename It2, typename T>
T inner_product(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2, T init) {
  using thrust::system::detail::generic::inner_product;
  return inner_product(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, init);
}
template <typename D, typename It1, typename It2, typename T, typename Op1, typename Op2>
T inner_product(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2, T init, Op1 op1,
                Op2 op2) {
  return inner_product(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, init, op1, op2);
}
template <typename It1, typename It2, typename T>
T inner_product(It1 first1, It1 last1, It2 first2, T init) {
  return thrust::inner_product(detail::policy_for<It1>(), first1, last1, first2, init);
}
template <typename It1, typename It2, typename T, typename Op1, typename Op2,
          typename = typename std::enable_if<!detail::is_execution_policy<It1>::value>::type>
T inner_product(It1 first1, It1 last1, It2 first2, T init, Op1 op1, Op2 op2) {
  return thrust::inner_product(detail::policy_for<It1>(), first1, last1, first2, init, op1, op2);
}

}  // namespace thrust
