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

#include <thrust/detail/minmax.h>
#include <thrust/functional.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/pair.h>
#include <thrust/reduce.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>
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
// An element and where it stands.  Positions are 32-bit while the range allows it: the pair is
// what every step of the reduction carries.
template <typename V, typename I>
struct located {
  V value;
  I index;
};
template <typename V, typename I>
struct locates {
  template <typename Tuple>
  __host__ __device__ located<V, I> operator()(const Tuple& t) const {
    located<V, I> r = {(V)thrust::get<0>(t), (I)thrust::get<1>(t)};
    return r;
  }
};
// Of two located elements the more extreme; of equivalent ones the earlier
// (thrust/system/detail/generic/extrema.inl:53-108).
template <typename V, typename I, typename Comp, bool LARGEST>
struct picks_extreme {
  mutable Comp comp;  // a caller's comparison need not be const-callable
  __host__ __device__ located<V, I> operator()(const located<V, I>& a, const located<V, I>& b) const {
    // selects, not branches: this runs once per element in the reduction's inner loop
    const bool a_before = comp(a.value, b.value), b_before = comp(b.value, a.value);
    const bool b_earlier = b.index < a.index;
    const bool take_b = LARGEST ? (a_before | (!b_before & b_earlier)) : (b_before | (!a_before & b_earlier));
    located<V, I> r;
    r.value = take_b ? b.value : a.value;
    r.index = take_b ? b.index : a.index;
    return r;
  }
};
// Both extremes in one pass.
template <typename V, typename I>
struct located_pair {
  located<V, I> smallest, largest;
};
template <typename V, typename I>
struct locates_pair {
  template <typename Tuple>
  __host__ __device__ located_pair<V, I> operator()(const Tuple& t) const {
    located<V, I> r = {(V)thrust::get<0>(t), (I)thrust::get<1>(t)};
    located_pair<V, I> p = {r, r};
    return p;
  }
};
template <typename V, typename I, typename Comp>
struct picks_both {
  mutable Comp comp;
  __host__ __device__ located_pair<V, I> operator()(const located_pair<V, I>& a, const located_pair<V, I>& b) const {
    const picks_extreme<V, I, Comp, false> lo = {comp};
    const picks_extreme<V, I, Comp, true> hi = {comp};
    located_pair<V, I> r = {lo(a.smallest, b.smallest), hi(a.largest, b.largest)};
    return r;
  }
};

// The range's first element on the host: what the reduction starts from.
template <typename V, typename D, typename It>
V first_value(execution_policy<D>& exec, It first) {
  void* stream = stream_of(exec);
  device_input<It> head(stream, temp_source_of(exec), first, 1);  // a computed element is written out first
  return read_scalar<V>(head.ptr(), stream, "extrema: first element");
}

template <bool LARGEST, typename I, typename D, typename It, typename Comp>
std::ptrdiff_t extreme_position(execution_policy<D>& exec, It first, std::ptrdiff_t n, Comp comp) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first, thrust::counting_iterator<I>(0)));
  const located<V, I> start = {first_value<V>(exec, first), 0};
  const picks_extreme<V, I, Comp, LARGEST> pick = {comp};
  const located<V, I> found = thrust::reduce(exec, thrust::make_transform_iterator(zipped, locates<V, I>()),
                                             thrust::make_transform_iterator(zipped + n, locates<V, I>()), start, pick);
  return (std::ptrdiff_t)found.index;
}
template <bool LARGEST, typename D, typename It, typename Comp>
It extreme_element(execution_policy<D>& exec, It first, It last, Comp comp) {
  if (first == last) return last;
  const std::ptrdiff_t n = last - first;
  return first + (n <= 0x7fffffff ? extreme_position<LARGEST, int>(exec, first, n, comp)
                                  : extreme_position<LARGEST, long long>(exec, first, n, comp));
}
template <typename I, typename D, typename It, typename Comp>
thrust::pair<It, It> both_extremes(execution_policy<D>& exec, It first, std::ptrdiff_t n, Comp comp) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first, thrust::counting_iterator<I>(0)));
  const located<V, I> one = {first_value<V>(exec, first), 0};
  const located_pair<V, I> start = {one, one};
  const picks_both<V, I, Comp> pick = {comp};
  const located_pair<V, I> found =
      thrust::reduce(exec, thrust::make_transform_iterator(zipped, locates_pair<V, I>()),
                     thrust::make_transform_iterator(zipped + n, locates_pair<V, I>()), start, pick);
  return thrust::pair<It, It>(first + (std::ptrdiff_t)found.smallest.index, first + (std::ptrdiff_t)found.largest.index);
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
  if (first == last) return thrust::pair<It, It>(last, last);
  const std::ptrdiff_t n = last - first;
  return n <= 0x7fffffff ? detail::both_extremes<int>(exec, first, n, comp)
                         : detail::both_extremes<long long>(exec, first, n, comp);
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
