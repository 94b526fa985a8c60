// thrust::lower_bound, upper_bound, binary_search, equal_range on a sorted range: for one value
// (an iterator, a bool, a pair of iterators) and for a range of values (positions or bools written
// to an output range), under operator< or a caller's strict weak order
// (thrust/system/detail/generic/binary_search.inl:40-460; testing/binary_search.cu,
// binary_search_vector.cu, binary_search_descending.cu, binary_search_vector_descending.cu).  What
// one does with a range after sorting it.  On the device system the vector forms are one
// element-wise pass in which every thread bisects the sorted range for its value (translation
// units compiled with hipcc), and the scalar forms are the vector forms of one value, as in the
// reference (binary_search.inl:181-226); the host system runs the standard bisections.
#pragma once
#include <algorithm>
#include <cstddef>

#include <thrust/device_vector.h>
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/transform.h>

namespace thrust {

template <typename D, typename It, typename VIt, typename Out, typename Comp>
Out lower_bound(const detail::execution_policy_base<D>& exec, It first, It last, VIt values_first, VIt values_last,
                Out output, Comp comp);
template <typename D, typename It, typename VIt, typename Out, typename Comp>
Out upper_bound(const detail::execution_policy_base<D>& exec, It first, It last, VIt values_first, VIt values_last,
                Out output, Comp comp);
template <typename D, typename It, typename VIt, typename Out, typename Comp>
Out binary_search(const detail::execution_policy_base<D>& exec, It first, It last, VIt values_first, VIt values_last,
                  Out output, Comp comp);

namespace system {
namespace cpp {
template <typename D, typename It, typename VIt, typename Out, typename Comp>
Out lower_bound(execution_policy<D>&, It first, It last, VIt values_first, VIt values_last, Out output, Comp comp) {
  for (; values_first != values_last; ++values_first, ++output) *output = std::lower_bound(first, last, *values_first, comp) - first;
  return output;
}
template <typename D, typename It, typename VIt, typename Out, typename Comp>
Out upper_bound(execution_policy<D>&, It first, It last, VIt values_first, VIt values_last, Out output, Comp comp) {
  for (; values_first != values_last; ++values_first, ++output) *output = std::upper_bound(first, last, *values_first, comp) - first;
  return output;
}
template <typename D, typename It, typename VIt, typename Out, typename Comp>
Out binary_search(execution_policy<D>&, It first, It last, VIt values_first, VIt values_last, Out output, Comp comp) {
  for (; values_first != values_last; ++values_first, ++output) *output = std::binary_search(first, last, *values_first, comp);
  return output;
}
template <typename D, typename It, typename T, typename Comp>
It lower_bound(execution_policy<D>&, It first, It last, const T& value, Comp comp) {
  return std::lower_bound(first, last, value, comp);
}
template <typename D, typename It, typename T, typename Comp>
It upper_bound(execution_policy<D>&, It first, It last, const T& value, Comp comp) {
  return std::upper_bound(first, last, value, comp);
}
template <typename D, typename It, typename T, typename Comp>
bool binary_search(execution_policy<D>&, It first, It last, const T& value, Comp comp) {
  return std::binary_search(first, last, value, comp);
}
}  // namespace cpp

namespace hip {
namespace detail {
// Bisection of range[0, n): the first position whose element is not before the value
// (UPPER: is after the value).
template <typename View, typename Comp, bool UPPER>
struct bisects {
  View range;
  long long n;
  mutable Comp comp;  // a caller's comparison need not be const-callable
  template <typename T>
  __host__ __device__ long long operator()(const T& value) const {
    long long lo = 0, hi = n;
    while (lo < hi) {
      const long long mid = lo + (hi - lo) / 2;
      const bool right = UPPER ? !comp(value, range[mid]) : (bool)comp(range[mid], value);
      if (right) lo = mid + 1;
      else hi = mid;
    }
    return lo;
  }
};
template <typename View, typename Comp>
struct contains_sorted {
  bisects<View, Comp, false> lower;
  template <typename T>
  __host__ __device__ bool operator()(const T& value) const {
    const long long at = lower(value);
    return at < lower.n && !lower.comp(value, lower.range[at]);
  }
};
}  // namespace detail

template <typename D, typename It, typename VIt, typename Out, typename Comp>
Out lower_bound(execution_policy<D>& exec, It first, It last, VIt values_first, VIt values_last, Out output, Comp comp) {
  typedef typename thrust::detail::device_view_of<It>::type View;
  const detail::bisects<View, Comp, false> f = {thrust::detail::device_view(first), (long long)(last - first), comp};
  return thrust::transform(exec, values_first, values_last, output, f);
}
template <typename D, typename It, typename VIt, typename Out, typename Comp>
Out upper_bound(execution_policy<D>& exec, It first, It last, VIt values_first, VIt values_last, Out output, Comp comp) {
  typedef typename thrust::detail::device_view_of<It>::type View;
  const detail::bisects<View, Comp, true> f = {thrust::detail::device_view(first), (long long)(last - first), comp};
  return thrust::transform(exec, values_first, values_last, output, f);
}
template <typename D, typename It, typename VIt, typename Out, typename Comp>
Out binary_search(execution_policy<D>& exec, It first, It last, VIt values_first, VIt values_last, Out output, Comp comp) {
  typedef typename thrust::detail::device_view_of<It>::type View;
  const detail::contains_sorted<View, Comp> f = {{thrust::detail::device_view(first), (long long)(last - first), comp}};
  return thrust::transform(exec, values_first, values_last, output, f);
}
// one value: the vector form over one element of device memory
template <typename D, typename It, typename T, typename Comp>
It lower_bound(execution_policy<D>& exec, It first, It last, const T& value, Comp comp) {
  thrust::device_vector<T> one(1, value);
  thrust::device_vector<long long> at(1);
  thrust::lower_bound(exec, first, last, one.begin(), one.end(), at.begin(), comp);
  return first + (std::ptrdiff_t)(long long)at[0];
}
template <typename D, typename It, typename T, typename Comp>
It upper_bound(execution_policy<D>& exec, It first, It last, const T& value, Comp comp) {
  thrust::device_vector<T> one(1, value);
  thrust::device_vector<long long> at(1);
  thrust::upper_bound(exec, first, last, one.begin(), one.end(), at.begin(), comp);
  return first + (std::ptrdiff_t)(long long)at[0];
}
template <typename D, typename It, typename T, typename Comp>
bool binary_search(execution_policy<D>& exec, It first, It last, const T& value, Comp comp) {
  thrust::device_vector<T> one(1, value);
  thrust::device_vector<int> found(1);
  thrust::binary_search(exec, first, last, one.begin(), one.end(), found.begin(), comp);
  return (int)found[0] != 0;
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry points: a range of values
#define THRUST_AMD_SEARCH_VECTOR_ENTRY(NAME)                                                                          \
  template <typename D, typename It, typename VIt, typename Out, typename Comp>                                       \
  Out NAME(const detail::execution_policy_base<D>& exec, It first, It last, VIt values_first, VIt values_last,        \
           Out output, Comp comp) {                                                                                   \
    return NAME(detail::derived_cast(detail::strip_const(exec)), first, last, values_first, values_last, output,      \
                comp);                                                                                                \
  }                                                                                                                   \
  template <typename D, typename It, typename VIt, typename Out>                                                      \
  Out NAME(const detail::execution_policy_base<D>& exec, It first, It last, VIt values_first, VIt values_last,        \
           Out output) {                                                                                              \
    typedef typename std::remove_const<typename iterator_value<It>::type>::type V;                                    \
    return thrust::NAME(exec, first, last, values_first, values_last, output, thrust::less<V>());                     \
  }                                                                                                                   \
  template <typename It, typename VIt, typename Out, typename Comp,                                                   \
            typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>                        \
  Out NAME(It first, It last, VIt values_first, VIt values_last, Out output, Comp comp) {                             \
    return thrust::NAME(detail::policy_for<It>(), first, last, values_first, values_last, output, comp);              \
  }                                                                                                                   \
  template <typename It, typename VIt, typename Out,                                                                  \
            typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>                        \
  Out NAME(It first, It last, VIt values_first, VIt values_last, Out output) {                                        \
    return thrust::NAME(detail::policy_for<It>(), first, last, values_first, values_last, output);                    \
  }
THRUST_AMD_SEARCH_VECTOR_ENTRY(lower_bound)
THRUST_AMD_SEARCH_VECTOR_ENTRY(upper_bound)
THRUST_AMD_SEARCH_VECTOR_ENTRY(binary_search)
#undef THRUST_AMD_SEARCH_VECTOR_ENTRY

// ------------------------------------------------------------------ entry points: one value
#define THRUST_AMD_SEARCH_SCALAR_ENTRY(NAME, RESULT)                                                                  \
  template <typename D, typename It, typename T, typename Comp>                                                       \
  RESULT NAME(const detail::execution_policy_base<D>& exec, It first, It last, const T& value, Comp comp) {           \
    return NAME(detail::derived_cast(detail::strip_const(exec)), first, last, value, comp);                           \
  }                                                                                                                   \
  template <typename D, typename It, typename T>                                                                      \
  RESULT NAME(const detail::execution_policy_base<D>& exec, It first, It last, const T& value) {                      \
    return thrust::NAME(exec, first, last, value, thrust::less<T>());                                                 \
  }                                                                                                                   \
  template <typename It, typename T, typename Comp,                                                                   \
            typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>                        \
  RESULT NAME(It first, It last, const T& value, Comp comp) {                                                         \
    return thrust::NAME(detail::policy_for<It>(), first, last, value, comp);                                          \
  }                                                                                                                   \
  template <typename It, typename T>                                                                                  \
  RESULT NAME(It first, It last, const T& value) {                                                                    \
    return thrust::NAME(detail::policy_for<It>(), first, last, value);                                                \
  }
THRUST_AMD_SEARCH_SCALAR_ENTRY(lower_bound, It)
THRUST_AMD_SEARCH_SCALAR_ENTRY(upper_bound, It)
THRUST_AMD_SEARCH_SCALAR_ENTRY(binary_search, bool)
#undef THRUST_AMD_SEARCH_SCALAR_ENTRY

template <typename D, typename It, typename T, typename Comp>
thrust::pair<It, It> equal_range(const detail::execution_policy_base<D>& exec, It first, It last, const T& value,
                                 Comp comp) {
  const It lower = thrust::lower_bound(exec, first, last, value, comp);
  return thrust::pair<It, It>(lower, thrust::upper_bound(exec, lower, last, value, comp));
}
template <typename D, typename It, typename T>
thrust::pair<It, It> equal_range(const detail::execution_policy_base<D>& exec, It first, It last, const T& value) {
  return thrust::equal_range(exec, first, last, value, thrust::less<T>());
}
template <typename It, typename T, typename Comp,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
thrust::pair<It, It> equal_range(It first, It last, const T& value, Comp comp) {
  return thrust::equal_range(detail::policy_for<It>(), first, last, value, comp);
}
template <typename It, typename T>
thrust::pair<It, It> equal_range(It first, It last, const T& value) {
  return thrust::equal_range(detail::policy_for<It>(), first, last, value);
}

}  // namespace thrust
