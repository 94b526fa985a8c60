// thrust::inner_product.
//
// inner_product(first1, last1, first2, init) = init + sum of a[i] * b[i]; the products
// and the sum are made in the type of init (multiplies<T> and plus<T>,
// thrust/system/detail/generic/inner_product.inl:33-65).  plus over multiplies on one arithmetic
// type runs in the library's kernel; any other pair of operators is a reduction over the zipped
// ranges (translation units compiled with hipcc).
#pragma once
#include <thrust/functional.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/reduce.h>
#include <thrust/tuple.h>

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
namespace detail {
// library path: two ranges and init of one arithmetic type, plus over multiplies
template <typename V1, typename V2, typename T, typename Op1, typename Op2, bool = is_abi_type<T>::value>
struct inner_product_in_library
    : std::integral_constant<bool, std::is_same<V1, T>::value && std::is_same<V2, T>::value &&
                                       binop_code<Op1, T>::value == THRUST_AMD_PLUS &&
                                       (std::is_same<Op2, thrust::multiplies<T> >::value ||
                                        std::is_same<Op2, thrust::multiplies<void> >::value)> {};
template <typename V1, typename V2, typename T, typename Op1, typename Op2>
struct inner_product_in_library<V1, V2, T, Op1, Op2, false> : std::false_type {};

// op2 on the two halves of a zipped element
template <typename Op2>
struct on_zipped_pair {
  mutable Op2 op;  // a caller's operator need not be const-callable
  template <typename Tuple>
  __host__ __device__ auto operator()(const Tuple& t) const -> decltype(op(thrust::get<0>(t), thrust::get<1>(t))) {
    return op(thrust::get<0>(t), thrust::get<1>(t));
  }
};

template <typename D, typename It1, typename It2, typename T, typename Op1, typename Op2>
T inner_product(execution_policy<D>& exec, It1 first1, It1 last1, It2 first2, T init, Op1, Op2, std::true_type) {
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last1 - first1);
  if (n == 0) return init;
  device_input<It1> source1(stream, temp_source_of(exec), first1, n);
  device_input<It2> source2(stream, temp_source_of(exec), first2, n);
  temp_storage temp(stream, temp_source_of(exec));
  void* d_out = nullptr;
  std::size_t need = 0;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_inner_product(t, b, source1.ptr(), source2.ptr(), n, dtype_of<T>::value, &init, d_out, stream);
  };
  throw_on_error(call(nullptr, &need), "inner_product: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_out = static_cast<char*>(temp.ptr()) + aligned;
  std::size_t bytes = aligned;
  throw_on_error(call(temp.ptr(), &bytes), "inner_product failed");
  return read_scalar<T>(d_out, stream, "inner_product: result copy");
}
// any two operators and element types: the reduction, under op1, of op2 over the zipped ranges
// (thrust/system/detail/generic/inner_product.inl:50-65)
template <typename D, typename It1, typename It2, typename T, typename Op1, typename Op2>
T inner_product(execution_policy<D>& exec, It1 first1, It1 last1, It2 first2, T init, Op1 op1, Op2 op2, std::false_type) {
#if defined(__HIPCC__)
  const on_zipped_pair<Op2> products = {op2};
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first1, first2));
  return thrust::reduce(exec, thrust::make_transform_iterator(zipped, products),
                        thrust::make_transform_iterator(zipped + (last1 - first1), products), init, op1);
#else
  static_assert(fancy_needs_hipcc<Op2>::value,
                "thrust::inner_product on the device system: operators other than thrust::plus over thrust::multiplies "
                "and mixed element types run in kernels instantiated for them; compile this translation unit with hipcc");
  return init;
#endif
}
}  // namespace detail

template <typename D, typename It1, typename It2, typename T, typename Op1, typename Op2>
T inner_product(execution_policy<D>& exec, It1 first1, It1 last1, It2 first2, T init, Op1 op1, Op2 op2) {
  typedef typename std::remove_const<typename iterator_value<It1>::type>::type V1;
  typedef typename std::remove_const<typename iterator_value<It2>::type>::type V2;
  static_assert(detail::is_device_input<It1>::value && detail::is_device_input<It2>::value,
                "thrust::inner_product on the device system needs device_ptr / device_vector iterators, raw device "
                "pointers or fancy iterators over them");
  return detail::inner_product(exec, first1, last1, first2, init, op1, op2,
                               detail::inner_product_in_library<V1, V2, T, Op1, Op2>());
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
