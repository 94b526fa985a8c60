// thrust::equal: two ranges agree element by element, under == or a caller's predicate
// (thrust/system/detail/generic/equal.inl:32-48: mismatch reaches the end; testing/equal.cu).
#pragma once
#include <thrust/mismatch.h>

namespace thrust {

template <typename D, typename It1, typename It2, typename Pred>
bool equal(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2, Pred pred) {
  return thrust::mismatch(exec, first1, last1, first2, pred).first == last1;
}
template <typename D, typename It1, typename It2>
bool equal(const detail::execution_policy_base<D>& exec, It1 first1, It1 last1, It2 first2) {
  typedef typename std::remove_const<typename iterator_value<It1>::type>::type V;
  return thrust::equal(exec, first1, last1, first2, thrust::equal_to<V>());
}
template <typename It1, typename It2, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<It1>::value>::type>
bool equal(It1 first1, It1 last1, It2 first2, Pred pred) {
  return thrust::equal(detail::policy_for<It1>(), first1, last1, first2, pred);
}
template <typename It1, typename It2>
bool equal(It1 first1, It1 last1, It2 first2) {
  return thrust::equal(detail::policy_for<It1>(), first1, last1, first2);
}

}  // namespace thrust
