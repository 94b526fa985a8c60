// thrust::inclusive_scan and thrust::exclusive_scan.
//
// Accumulator types follow the reference (thrust/system/detail/sequential/scan.h:48-115,
// P0571): inclusive scans accumulate in the input's value type, exclusive scans in the
// type of init; exclusive_scan(first,last,result) uses init = value_type(0); the default
// operator is plus (thrust/system/detail/generic/scan.inl:39-81).  In-place is allowed.
#pragma once
#include <thrust/functional.h>
#include <thrust/system/hip/detail/backend.h>

namespace thrust {

template <typename D, typename In, typename Out>
Out inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result);
template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Op op);
template <typename D, typename In, typename Out>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result);
template <typename D, typename In, typename Out, typename T>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, T init);
template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, T init, Op op);

namespace system {
namespace detail {
namespace generic {
template <typename D, typename In, typename Out>
Out inclusive_scan(thrust::execution_policy<D>& exec, In first, In last, Out result) {
  return thrust::inclusive_scan(exec, first, last, result, thrust::plus<>());
}
template <typename D, typename In, typename Out>
Out exclusive_scan(thrust::execution_policy<D>& exec, In first, In last, Out result) {
  typedef typename iterator_value<In>::type T;
  return thrust::exclusive_scan(exec, first, last, result, T(0));
}
template <typename D, typename In, typename Out, typename T>
Out exclusive_scan(thrust::execution_policy<D>& exec, In first, In last, Out result, T init) {
  return thrust::exclusive_scan(exec, first, last, result, init, thrust::plus<>());
}
}  // namespace generic
}  // namespace detail

namespace cpp {
template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(execution_policy<D>&, In first, In last, Out result, Op op) {
  typedef typename iterator_value<In>::type T;
  if (first != last) {
    T sum = *first;
    *result = sum;
    for (++first, ++result; first != last; ++first, ++result) *result = sum = op(sum, *first);
  }
  return result;
}
template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(execution_policy<D>&, In first, In last, Out result, T init, Op op) {
  if (first != last) {
    T tmp = *first;
    T sum = init;
    *result = sum;
    sum = op(sum, tmp);
    for (++first, ++result; first != last; ++first, ++result) {
      tmp = *first;
      *result = sum;
      sum = op(sum, tmp);
    }
  }
  return result;
}
}  // namespace cpp

namespace hip {
namespace detail {
template <typename In, typename Out, typename T, typename Op>
struct scan_checks {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  static_assert((std::is_pointer<In>::value || thrust::detail::is_device_iterator<In>::value) &&
                    (std::is_pointer<Out>::value || thrust::detail::is_device_iterator<Out>::value),
                "scan on the device system needs device_ptr / device_vector iterators or raw device pointers");
  static_assert(is_abi_type<V>::value && std::is_same<V, T>::value &&
                    std::is_same<typename iterator_value<Out>::type, V>::value,
                "scan on the device system: input, output and init must share one arithmetic type");
  static_assert(binop_code<Op, V>::value >= 0,
                "scan on the device system supports thrust::plus, thrust::minimum and thrust::maximum");
};
}  // namespace detail

template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Op) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  (void)sizeof(detail::scan_checks<In, Out, V, Op>);
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  detail::temp_storage temp(stream);
  detail::run(temp, 0, "inclusive_scan failed", [&](void* t, std::size_t* b) {
    return thrust_amd_inclusive_scan(t, b, thrust::detail::raw(first), thrust::detail::raw(result), n,
                                     detail::dtype_of<V>::value, detail::binop_code<Op, V>::value, stream);
  });
  detail::synchronize(stream, "inclusive_scan: synchronize");
  return result + n;
}

template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(execution_policy<D>& exec, In first, In last, Out result, T init, Op) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  (void)sizeof(detail::scan_checks<In, Out, T, Op>);
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  detail::temp_storage temp(stream);
  detail::run(temp, 0, "exclusive_scan failed", [&](void* t, std::size_t* b) {
    return thrust_amd_exclusive_scan(t, b, thrust::detail::raw(first), thrust::detail::raw(result), n,
                                     detail::dtype_of<V>::value, detail::binop_code<Op, V>::value, &init, stream);
  });
  detail::synchronize(stream, "exclusive_scan: synchronize");
  return result + n;
}
}  // namespace hip
}  // namespace system

template <typename D, typename In, typename Out>
Out inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  using thrust::system::detail::generic::inclusive_scan;
  return inclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Op op) {
  using thrust::system::detail::generic::inclusive_scan;
  return inclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, op);
}
template <typename D, typename In, typename Out>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  using thrust::system::detail::generic::exclusive_scan;
  return exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
template <typename D, typename In, typename Out, typename T>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, T init) {
  using thrust::system::detail::generic::exclusive_scan;
  return exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, init);
}
template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, T init, Op op) {
  using thrust::system::detail::generic::exclusive_scan;
  return exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, init, op);
}

template <typename In, typename Out>
Out inclusive_scan(In first, In last, Out result) {
  return thrust::inclusive_scan(detail::policy_for<In>(), first, last, result);
}
template <typename In, typename Out, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out inclusive_scan(In first, In last, Out result, Op op) {
  return thrust::inclusive_scan(detail::policy_for<In>(), first, last, result, op);
}
template <typename In, typename Out>
Out exclusive_scan(In first, In last, Out result) {
  return thrust::exclusive_scan(detail::policy_for<In>(), first, last, result);
}
template <typename In, typename Out, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out exclusive_scan(In first, In last, Out result, T init) {
  return thrust::exclusive_scan(detail::policy_for<In>(), first, last, result, init);
}
template <typename In, typename Out, typename T, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out exclusive_scan(In first, In last, Out result, T init, Op op) {
  return thrust::exclusive_scan(detail::policy_for<In>(), first, last, result, init, op);
}

}  // namespace thrust
