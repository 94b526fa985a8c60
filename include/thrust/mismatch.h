// thrust::mismatch: the first position where two ranges differ (or where the predicate that
// relates them fails), as a pair of iterators; (last1, first2 + n) when they agree throughout
// (thrust/system/detail/generic/mismatch.inl:37-71; testing/mismatch.cu).  A find_if over the
// zipped ranges.
#pragma once
#include <cstddef>

#include <thrust/find.h>
#include <thrust/functional.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/pair.h>
#include <thrust/tuple.h>

namespace thrust {
namespace detail {
template <typename Pred>
struct pair_fails {
  mutable Pred pred;
  template <typename Tuple>
  __host__ __device__ bool operator()(const Tuple& t) const { return !pred(thrust::get<0>(t), thrust::get<1>(t)); }
};
}  // namespace detail

template <typename D, typename It1, typename It2, typename Pred>
thrust::pair<It1, It2> mismatch(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2,
                                Pred pred) {
  const std::ptrdiff_t n = last1 - first1;
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first1, first2));
  const detail::pair_fails<Pred> fails = {pred};
  const std::ptrdiff_t at = thrust::find_if(exec, zipped, zipped + n, fails) - zipped;
  return thrust::pair<It1, It2>(first1 + at, first2 + at);
}
template <typename D, typename It1, typename It2>
thrust::pair<It1, It2> mismatch(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2) {
  typedef typename std::remove_const<typename iterator_value<It1>::type>::type V;
  return thrust::mismatch(exec, first1, last1, first2, thrust::equal_to<V>());
}
template <typename It1, typename It2, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<It1>::value>::type>
thrust::pair<It1, It2> mismatch(It1 first1, It1 last1, It2 first2, Pred pred) {
  return thrust::mismatch(detail::policy_for<It1>(), first1, last1, first2, pred);
}
template <typename It1, typename It2>
thrust::pair<It1, It2> mismatch(It1 first1, It1 last1, It2 first2) {
  return thrust::mismatch(detail::policy_for<It1>(), first1, last1, first2);
}

}  // namespace thrust
