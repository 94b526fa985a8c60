// thrust::find, thrust::find_if, thrust::find_if_not.
//
// The first position whose element equals a value / satisfies (does not satisfy) a predicate,
// `last` when there is none (thrust/system/detail/generic/find.inl:39-149; testing/find.cu).  On
// the device system: the smallest position among the elements that qualify, one reduction with
// thrust::minimum over positions (the reference reduces interval by interval and stops early;
// this reads the range once).  Translation units compiled with hipcc; the host system runs the
// sequential loop.
#pragma once
#include <cstddef>

#include <thrust/functional.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/reduce.h>
#include <thrust/tuple.h>

namespace thrust {

template <typename D, typename It, typename Pred>
It find_if(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred);

namespace detail {
// x == value, compared as the reference does (thrust/detail/internal_functional.h: equal_to_value)
template <typename T>
struct equals_value {
  T value;
  template <typename V>
  __host__ __device__ bool operator()(const V& x) const { return x == value; }
};
template <typename Pred>
struct negated {
  mutable Pred pred;  // a caller's predicate need not be const-callable
  template <typename V>
  __host__ __device__ bool operator()(const V& x) const { return !pred(x); }
};
// (element, position) -> position if the element qualifies, else `none`
template <typename Pred>
struct position_if {
  mutable Pred pred;
  long long none;
  template <typename Tuple>
  __host__ __device__ long long operator()(const Tuple& t) const {
    return pred(thrust::get<0>(t)) ? (long long)thrust::get<1>(t) : none;
  }
};
}  // namespace detail

namespace system {
namespace cpp {
template <typename D, typename It, typename Pred>
It find_if(execution_policy<D>&, It first, It last, Pred pred) {
  for (; first != last; ++first)
    if (pred(*first)) return first;
  return last;
}
}  // namespace cpp

namespace hip {
template <typename D, typename It, typename Pred>
It find_if(execution_policy<D>& exec, It first, It last, Pred pred) {
  if (first == last) return last;
  const long long n = (long long)(last - first);
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first, thrust::counting_iterator<long long>(0)));
  const thrust::detail::position_if<Pred> where = {pred, n};
  const long long at = thrust::reduce(exec, thrust::make_transform_iterator(zipped, where),
                                      thrust::make_transform_iterator(zipped + (std::ptrdiff_t)n, where), n,
                                      thrust::minimum<long long>());
  return first + (std::ptrdiff_t)at;
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry points
template <typename D, typename It, typename Pred>
It find_if(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return find_if(detail::derived_cast(detail::strip_const(exec)), first, last, pred);
}
template <typename D, typename It, typename Pred>
It find_if_not(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  const detail::negated<Pred> not_pred = {pred};
  return thrust::find_if(exec, first, last, not_pred);
}
template <typename D, typename It, typename T>
It find(const detail::execution_policy_base<D>& exec, It first, It last, const T& value) {
  const detail::equals_value<T> is_value = {value};
  return thrust::find_if(exec, first, last, is_value);
}
template <typename It, typename Pred, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It find_if(It first, It last, Pred pred) {
  return thrust::find_if(detail::policy_for<It>(), first, last, pred);
}
template <typename It, typename Pred, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It find_if_not(It first, It last, Pred pred) {
  return thrust::find_if_not(detail::policy_for<It>(), first, last, pred);
}
template <typename It, typename T, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It find(It first, It last, const T& value) {
  return thrust::find(detail::policy_for<It>(), first, last, value);
}

}  // namespace thrust
