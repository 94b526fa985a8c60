// thrust::min_element, thrust::max_element, thrust::minmax_element.
//
// The position of the smallest / largest element under operator< or a caller's strict weak
// order; of equivalent extremes the first one (both in minmax_element), and `last` for an empty
// range (thrust/system/detail/generic/extrema.inl:53-122 the tie rules, :150-247 the drivers;
// testing/min_element.cu, max_element.cu, minmax_element.cu).  On the device system this is one
// reduction over (element, position) pairs: the caller of thrust::reduce on the side of the
// path that looks for where, not for how much (translation units compiled with hipcc); the host
// system runs the sequential loop.
#pragma once
#include <cstddef>

#include <thrust/functional.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/pair.h>
#include <thrust/reduce.h>
#include <thrust/tuple.h>

namespace thrust {

template <typename D, typename It, typename Comp>
It min_element(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp);
template <typename D, typename It, typename Comp>
It max_element(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp);
template <typename D, typename It, typename Comp>
thrust::pair<It, It> minmax_element(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp);

namespace system {
namespace cpp {
template <typename D, typename It, typename Comp>
It min_element(execution_policy<D>&, It first, It last, Comp comp) {
  if (first == last) return last;
  It best = first;
  for (It it = first; ++it != last;)
    if (comp(*it, *best)) best = it;
  return best;
}
template <typename D, typename It, typename Comp>
It max_element(execution_policy<D>&, It first, It last, Comp comp) {
  if (first == last) return last;
  It best = first;
  for (It it = first; ++it != last;)
    if (comp(*best, *it)) best = it;
  return best;
}
template <typename D, typename It, typename Comp>
thrust::pair<It, It> minmax_element(execution_policy<D>& exec, It first, It last, Comp comp) {
  return thrust::pair<It, It>(min_element(exec, first, last, comp), max_element(exec, first, last, comp));
}
}  // namespace cpp

namespace hip {
namespace detail {
// An element and where it stands; index < 0: nothing seen yet.
template <typename V>
struct located {
  V value;
  long long index;
};
template <typename V>
struct locates {
  template <typename Tuple>
  __host__ __device__ located<V> operator()(const Tuple& t) const {
    located<V> r = {(V)thrust::get<0>(t), (long long)thrust::get<1>(t)};
    return r;
  }
};
// Of two located elements the more extreme; of equivalent ones the earlier.
template <typename V, typename Comp, bool LARGEST>
struct picks_extreme {
  mutable Comp comp;  // a caller's comparison need not be const-callable
  __host__ __device__ located<V> operator()(const located<V>& a, const located<V>& b) const {
    if (a.index < 0) return b;
    if (b.index < 0) return a;
    const bool a_first = a.index < b.index;
    const located<V>& early = a_first ? a : b;
    const located<V>& late = a_first ? b : a;
    const bool late_wins = LARGEST ? (bool)comp(early.value, late.value) : (bool)comp(late.value, early.value);
    return late_wins ? late : early;
  }
};
// Both extremes in one pass.
template <typename V>
struct located_pair {
  located<V> smallest, largest;
};
template <typename V>
struct locates_pair {
  template <typename Tuple>
  __host__ __device__ located_pair<V> operator()(const Tuple& t) const {
    located<V> r = {(V)thrust::get<0>(t), (long long)thrust::get<1>(t)};
    located_pair<V> p = {r, r};
    return p;
  }
};
template <typename V, typename Comp>
struct picks_both {
  Comp comp;
  __host__ __device__ located_pair<V> operator()(const located_pair<V>& a, const located_pair<V>& b) const {
    const picks_extreme<V, Comp, false> lo = {comp};
    const picks_extreme<V, Comp, true> hi = {comp};
    located_pair<V> r = {lo(a.smallest, b.smallest), hi(a.largest, b.largest)};
    return r;
  }
};

template <bool LARGEST, typename D, typename It, typename Comp>
It extreme_element(execution_policy<D>& exec, It first, It last, Comp comp) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  if (first == last) return last;
  const std::ptrdiff_t n = last - first;
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first, thrust::counting_iterator<long long>(0)));
  const located<V> nothing = {V(), -1};
  const picks_extreme<V, Comp, LARGEST> pick = {comp};
  const located<V> found = thrust::reduce(exec, thrust::make_transform_iterator(zipped, locates<V>()),
                                          thrust::make_transform_iterator(zipped + n, locates<V>()), nothing, pick);
  return first + (std::ptrdiff_t)found.index;
}
}  // namespace detail

template <typename D, typename It, typename Comp>
It min_element(execution_policy<D>& exec, It first, It last, Comp comp) {
  return detail::extreme_element<false>(exec, first, last, comp);
}
template <typename D, typename It, typename Comp>
It max_element(execution_policy<D>& exec, It first, It last, Comp comp) {
  return detail::extreme_element<true>(exec, first, last, comp);
}
template <typename D, typename It, typename Comp>
thrust::pair<It, It> minmax_element(execution_policy<D>& exec, It first, It last, Comp comp) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  if (first == last) return thrust::pair<It, It>(last, last);
  const std::ptrdiff_t n = last - first;
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first, thrust::counting_iterator<long long>(0)));
  const detail::located<V> nothing = {V(), -1};
  const detail::located_pair<V> none = {nothing, nothing};
  const detail::picks_both<V, Comp> pick = {comp};
  const detail::located_pair<V> found =
      thrust::reduce(exec, thrust::make_transform_iterator(zipped, detail::locates_pair<V>()),
                     thrust::make_transform_iterator(zipped + n, detail::locates_pair<V>()), none, pick);
  return thrust::pair<It, It>(first + (std::ptrdiff_t)found.smallest.index, first + (std::ptrdiff_t)found.largest.index);
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry points
template <typename D, typename It, typename Comp>
It min_element(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp) {
  return min_element(detail::derived_cast(detail::strip_const(exec)), first, last, comp);
}
template <typename D, typename It>
It min_element(const detail::execution_policy_base<D>& exec, It first, It last) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  return thrust::min_element(exec, first, last, thrust::less<V>());
}
template <typename It, typename Comp, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It min_element(It first, It last, Comp comp) {
  return thrust::min_element(detail::policy_for<It>(), first, last, comp);
}
template <typename It>
It min_element(It first, It last) {
  return thrust::min_element(detail::policy_for<It>(), first, last);
}

template <typename D, typename It, typename Comp>
It max_element(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp) {
  return max_element(detail::derived_cast(detail::strip_const(exec)), first, last, comp);
}
template <typename D, typename It>
It max_element(const detail::execution_policy_base<D>& exec, It first, It last) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  return thrust::max_element(exec, first, last, thrust::less<V>());
}
template <typename It, typename Comp, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It max_element(It first, It last, Comp comp) {
  return thrust::max_element(detail::policy_for<It>(), first, last, comp);
}
template <typename It>
It max_element(It first, It last) {
  return thrust::max_element(detail::policy_for<It>(), first, last);
}

template <typename D, typename It, typename Comp>
thrust::pair<It, It> minmax_element(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp) {
  return minmax_element(detail::derived_cast(detail::strip_const(exec)), first, last, comp);
}
template <typename D, typename It>
thrust::pair<It, It> minmax_element(const detail::execution_policy_base<D>& exec, It first, It last) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  return thrust::minmax_element(exec, first, last, thrust::less<V>());
}
template <typename It, typename Comp, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
thrust::pair<It, It> minmax_element(It first, It last, Comp comp) {
  return thrust::minmax_element(detail::policy_for<It>(), first, last, comp);
}
template <typename It>
thrust::pair<It, It> minmax_element(It first, It last) {
  return thrust::minmax_element(detail::policy_for<It>(), first, last);
}

}  // namespace thrust
