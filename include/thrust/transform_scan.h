// thrust::transform_inclusive_scan and thrust::transform_exclusive_scan.
//
// The scans of thrust/scan.h over unary_op(x) instead of x.  The running value has the
// type unary_op returns (inclusive form) or the type of init (exclusive form)
// (thrust/system/detail/generic/transform_scan.inl:37-97).  On the device system unary_op
// is one of thrust::identity / negate / square on the element type and binary_op one of
// plus / minimum / maximum; result may be the input range.
#pragma once
#include <thrust/functional.h>
#include <thrust/system/hip/detail/backend.h>

namespace thrust {

template <typename D, typename In, typename Out, typename Fn, typename Op>
Out transform_inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Fn unary_op,
                             Op binary_op);
template <typename D, typename In, typename Out, typename Fn, typename T, typename Op>
Out transform_exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Fn unary_op,
                             T init, Op binary_op);

namespace system {
namespace cpp {
// sequential scans (thrust/system/detail/sequential/scan.h:48-115) reading through unary_op
template <typename D, typename In, typename Out, typename Fn, typename Op>
Out transform_inclusive_scan(execution_policy<D>&, In first, In last, Out result, Fn unary_op, Op binary_op) {
  typedef typename std::decay<decltype(unary_op(*first))>::type T;
  if (first != last) {
    T sum = unary_op(*first);
    *result = sum;
    for (++first, ++result; first != last; ++first, ++result) *result = sum = binary_op(sum, static_cast<T>(unary_op(*first)));
  }
  return result;
}
template <typename D, typename In, typename Out, typename Fn, typename T, typename Op>
Out transform_exclusive_scan(execution_policy<D>&, In first, In last, Out result, Fn unary_op, T init, Op binary_op) {
  if (first != last) {
    T tmp = static_cast<T>(unary_op(*first));
    T sum = init;
    *result = sum;
    sum = binary_op(sum, tmp);
    for (++first, ++result; first != last; ++first, ++result) {
      tmp = static_cast<T>(unary_op(*first));
      *result = sum;
      sum = binary_op(sum, tmp);
    }
  }
  return result;
}
}  // namespace cpp

namespace hip {
namespace detail {
template <typename In, typename Out, typename T, typename Fn, typename Op>
struct transform_scan_checks {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  static_assert((std::is_pointer<In>::value || thrust::detail::is_device_iterator<In>::value) &&
                    (std::is_pointer<Out>::value || thrust::detail::is_device_iterator<Out>::value),
                "transform scans on the device system need device_ptr / device_vector iterators or raw device pointers");
  static_assert(is_abi_type<V>::value && std::is_same<V, T>::value &&
                    std::is_same<typename iterator_value<Out>::type, V>::value,
                "transform scans on the device system: input, output and init must share one arithmetic type");
  static_assert(unary_code<Fn, V>::value >= 0,
                "transform scans on the device system support thrust::identity, thrust::negate and thrust::square");
  static_assert(binop_code<Op, V>::value >= 0,
                "transform scans on the device system support thrust::plus, thrust::minimum and thrust::maximum");
};
}  // namespace detail

template <typename D, typename In, typename Out, typename Fn, typename Op>
Out transform_inclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Fn, Op) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  (void)sizeof(detail::transform_scan_checks<In, Out, V, Fn, Op>);
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  detail::temp_storage temp(stream, detail::temp_source_of(exec));
  detail::run(temp, 0, "transform_inclusive_scan failed", [&](void* t, std::size_t* b) {
    return thrust_amd_transform_inclusive_scan(t, b, thrust::detail::raw(first), thrust::detail::raw(result), n,
                                               detail::dtype_of<V>::value, detail::unary_code<Fn, V>::value,
                                               detail::binop_code<Op, V>::value, stream);
  });
  detail::synchronize(stream, "transform_inclusive_scan: synchronize");
  return result + n;
}

template <typename D, typename In, typename Out, typename Fn, typename T, typename Op>
Out transform_exclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Fn, T init, Op) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  (void)sizeof(detail::transform_scan_checks<In, Out, T, Fn, Op>);
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  detail::temp_storage temp(stream, detail::temp_source_of(exec));
  detail::run(temp, 0, "transform_exclusive_scan failed", [&](void* t, std::size_t* b) {
    return thrust_amd_transform_exclusive_scan(t, b, thrust::detail::raw(first), thrust::detail::raw(result), n,
                                               detail::dtype_of<V>::value, detail::unary_code<Fn, V>::value,
                                               detail::binop_code<Op, V>::value, &init, stream);
  });
  detail::synchronize(stream, "transform_exclusive_scan: synchronize");
  return result + n;
}
}  // namespace hip
}  // namespace system

template <typename D, typename In, typename Out, typename Fn, typename Op>
Out transform_inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Fn unary_op,
                             Op binary_op) {
  return transform_inclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, unary_op,
                                  binary_op);
}
template <typename D, typename In, typename Out, typename Fn, typename T, typename Op>
Out transform_exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Fn unary_op,
                             T init, Op binary_op) {
  return transform_exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, unary_op, init,
                                  binary_op);
}
template <typename In, typename Out, typename Fn, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out transform_inclusive_scan(In first, In last, Out result, Fn unary_op, Op binary_op) {
  return thrust::transform_inclusive_scan(detail::policy_for<In>(), first, last, result, unary_op, binary_op);
}
template <typename In, typename Out, typename Fn, typename T, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out transform_exclusive_scan(In first, In last, Out result, Fn unary_op, T init, Op binary_op) {
  return thrust::transform_exclusive_scan(detail::policy_for<In>(), first, last, result, unary_op, init, binary_op);
}

}  // namespace thrust
