// thrust::all_of, thrust::any_of, thrust::none_of (thrust/system/detail/generic/logical.h:35-58:
// all_of = no element fails, any_of = some element passes, none_of = not any_of; an empty range
// gives true, false, true; testing/logical.cu).  Callers of find_if.
#pragma once
#include <thrust/find.h>

namespace thrust {

template <typename D, typename It, typename Pred>
bool all_of(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return thrust::find_if_not(exec, first, last, pred) == last;
}
template <typename D, typename It, typename Pred>
bool any_of(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return thrust::find_if(exec, first, last, pred) != last;
}
template <typename D, typename It, typename Pred>
bool none_of(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return !thrust::any_of(exec, first, last, pred);
}
template <typename It, typename Pred, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
bool all_of(It first, It last, Pred pred) {
  return thrust::all_of(detail::policy_for<It>(), first, last, pred);
}
template <typename It, typename Pred, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
bool any_of(It first, It last, Pred pred) {
  return thrust::any_of(detail::policy_for<It>(), first, last, pred);
}
template <typename It, typename Pred, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
bool none_of(It first, It last, Pred pred) {
  return thrust::none_of(detail::policy_for<It>(), first, last, pred);
}

}  // namespace thrust
