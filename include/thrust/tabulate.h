// thrust::tabulate: x[i] = op(i) (thrust/system/detail/generic/tabulate.inl:33-52: a transform of
// a counting iterator; testing/tabulate.cu).
#pragma once
#include <cstddef>

#include <thrust/iterator/counting_iterator.h>
#include <thrust/transform.h>

namespace thrust {

template <typename D, typename It, typename Op>
void tabulate(const detail::execution_policy_base<D>& exec, It first, It last, Op op) {
  typedef std::ptrdiff_t Index;
  thrust::counting_iterator<Index> zero(0);
  thrust::transform(exec, zero, zero + (last - first), first, op);
}
template <typename It, typename Op, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void tabulate(It first, It last, Op op) {
  thrust::tabulate(detail::policy_for<It>(), first, last, op);
}

}  // namespace thrust
