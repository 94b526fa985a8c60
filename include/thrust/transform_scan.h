// thrust::transform_inclusive_scan and thrust::transform_exclusive_scan.
//
// The scans of thrust/scan.h over unary_op(x) instead of x.  The running value has the
// type unary_op returns (inclusive form) or the type of init (exclusive form)
// (thrust/system/detail/generic/transform_scan.inl:37-97).  On the device system
// thrust::identity / negate / square with plus / minimum / maximum over arrays of one
// arithmetic type run in the library's scan kernel; any other function, operator, iterator or
// mix of types is the scan of a transform iterator (translation units compiled with hipcc).
// result may be the input range.
#pragma once
#include <thrust/functional.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/scan.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/staged_output.h>

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
// library path: arrays of one arithmetic type in and out, identity / negate / square, plus /
// minimum / maximum
template <typename In, typename Out, typename T, typename Fn, typename Op,
          bool = is_abi_type<typename std::remove_const<typename iterator_value<In>::type>::type>::value>
struct transform_scans_in_library
    : std::integral_constant<
          bool, is_memory_iterator<In>::value && is_memory_iterator<Out>::value &&
                    std::is_same<typename std::remove_const<typename iterator_value<In>::type>::type, T>::value &&
                    std::is_same<typename iterator_value<Out>::type, T>::value &&
                    (unary_code<Fn, typename std::remove_const<typename iterator_value<In>::type>::type>::value >= 0) &&
                    (binop_code<Op, typename std::remove_const<typename iterator_value<In>::type>::type>::value >= 0)> {};
template <typename In, typename Out, typename T, typename Fn, typename Op>
struct transform_scans_in_library<In, Out, T, Fn, Op, false> : std::false_type {};

template <typename D, typename In, typename Out, typename Fn, typename Op>
Out transform_inclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Fn, Op, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  temp_storage temp(stream, temp_source_of(exec));
  run(temp, 0, "transform_inclusive_scan failed", [&](void* t, std::size_t* b) {
    return thrust_amd_transform_inclusive_scan(t, b, thrust::detail::raw(first), thrust::detail::raw(result), n,
                                               dtype_of<V>::value, unary_code<Fn, V>::value, binop_code<Op, V>::value,
                                               stream);
  });
  synchronize(stream, "transform_inclusive_scan: synchronize");
  return result + n;
}
template <typename D, typename In, typename Out, typename Fn, typename T, typename Op>
Out transform_exclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Fn, T init, Op, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  temp_storage temp(stream, temp_source_of(exec));
  run(temp, 0, "transform_exclusive_scan failed", [&](void* t, std::size_t* b) {
    return thrust_amd_transform_exclusive_scan(t, b, thrust::detail::raw(first), thrust::detail::raw(result), n,
                                               dtype_of<V>::value, unary_code<Fn, V>::value, binop_code<Op, V>::value,
                                               &init, stream);
  });
  synchronize(stream, "transform_exclusive_scan: synchronize");
  return result + n;
}
// Everything else is the scan of a transform iterator, as the reference's generic layer states
// it (thrust/system/detail/generic/transform_scan.inl:37-97): any function, any operator, fancy
// inputs, outputs of another type or that are not memory.
template <typename D, typename In, typename Out, typename Fn, typename Op>
Out transform_inclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Fn unary_op, Op binary_op,
                             std::false_type) {
#if defined(__HIPCC__)
  return thrust::inclusive_scan(exec, thrust::make_transform_iterator(first, unary_op),
                                thrust::make_transform_iterator(last, unary_op), result, binary_op);
#else
  static_assert(fancy_needs_hipcc<Fn>::value,
                "transform scans on the device system: functions other than thrust::identity / negate / square, operators "
                "other than thrust::plus / minimum / maximum, fancy iterators and mixed element types run in kernels "
                "instantiated for them; compile this translation unit with hipcc");
  return result;
#endif
}
template <typename D, typename In, typename Out, typename Fn, typename T, typename Op>
Out transform_exclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Fn unary_op, T init, Op binary_op,
                             std::false_type) {
#if defined(__HIPCC__)
  return thrust::exclusive_scan(exec, thrust::make_transform_iterator(first, unary_op),
                                thrust::make_transform_iterator(last, unary_op), result, init, binary_op);
#else
  static_assert(fancy_needs_hipcc<Fn>::value,
                "transform scans on the device system: functions other than thrust::identity / negate / square, operators "
                "other than thrust::plus / minimum / maximum, fancy iterators and mixed element types run in kernels "
                "instantiated for them; compile this translation unit with hipcc");
  return result;
#endif
}
}  // namespace detail

template <typename D, typename In, typename Out, typename Fn, typename Op>
Out transform_inclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Fn unary_op, Op binary_op) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  return detail::transform_inclusive_scan(exec, first, last, result, unary_op, binary_op,
                                          detail::transform_scans_in_library<In, Out, V, Fn, Op>());
}
template <typename D, typename In, typename Out, typename Fn, typename T, typename Op>
Out transform_exclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Fn unary_op, T init, Op binary_op) {
  return detail::transform_exclusive_scan(exec, first, last, result, unary_op, init, binary_op,
                                          detail::transform_scans_in_library<In, Out, T, Fn, Op>());
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
