// thrust::replace, replace_if, replace_copy, replace_copy_if (with and without a stencil):
// elements that equal a value / whose element or stencil satisfies a predicate become new_value
// (thrust/system/detail/generic/replace.inl:33-168; testing/replace.cu).  Element-wise transforms.
#pragma once
#include <thrust/find.h>
#include <thrust/functional.h>
#include <thrust/transform.h>

namespace thrust {
namespace detail {
template <typename Pred, typename T>
struct new_value_if {
  mutable Pred pred;  // a caller's predicate need not be const-callable
  T new_value;
  template <typename V>
  __host__ __device__ T operator()(const V& x) const { return pred(x) ? new_value : (T)x; }
  template <typename V, typename S>
  __host__ __device__ T operator()(const V& x, const S& stencil) const { return pred(stencil) ? new_value : (T)x; }
};
}  // namespace detail

template <typename D, typename In, typename Out, typename Pred, typename T>
Out replace_copy_if(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Pred pred,
                    const T& new_value) {
  typedef typename std::remove_const<typename iterator_value<Out>::type>::type U;
  const detail::new_value_if<Pred, U> f = {pred, (U)new_value};
  return thrust::transform(exec, first, last, result, f);
}
template <typename D, typename In, typename St, typename Out, typename Pred, typename T>
Out replace_copy_if(const detail::execution_policy_base<D>& exec, In first, In last, St stencil, Out result, Pred pred,
                    const T& new_value) {
  typedef typename std::remove_const<typename iterator_value<Out>::type>::type U;
  const detail::new_value_if<Pred, U> f = {pred, (U)new_value};
  return thrust::transform(exec, first, last, stencil, result, f);
}
template <typename D, typename In, typename Out, typename T>
Out replace_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result, const T& old_value,
                 const T& new_value) {
  const detail::equals_value<T> is_old = {old_value};
  return thrust::replace_copy_if(exec, first, last, result, is_old, new_value);
}
template <typename D, typename It, typename Pred, typename T>
void replace_if(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred, const T& new_value) {
  thrust::replace_copy_if(exec, first, last, first, pred, new_value);
}
template <typename D, typename It, typename St, typename Pred, typename T>
void replace_if(const detail::execution_policy_base<D>& exec, It first, It last, St stencil, Pred pred,
                const T& new_value) {
  thrust::replace_copy_if(exec, first, last, stencil, first, pred, new_value);
}
template <typename D, typename It, typename T>
void replace(const detail::execution_policy_base<D>& exec, It first, It last, const T& old_value, const T& new_value) {
  thrust::replace_copy(exec, first, last, first, old_value, new_value);
}

template <typename In, typename Out, typename Pred, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out replace_copy_if(In first, In last, Out result, Pred pred, const T& new_value) {
  return thrust::replace_copy_if(detail::policy_for<Out>(), first, last, result, pred, new_value);
}
template <typename In, typename St, typename Out, typename Pred, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out replace_copy_if(In first, In last, St stencil, Out result, Pred pred, const T& new_value) {
  return thrust::replace_copy_if(detail::policy_for<Out>(), first, last, stencil, result, pred, new_value);
}
template <typename In, typename Out, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out replace_copy(In first, In last, Out result, const T& old_value, const T& new_value) {
  return thrust::replace_copy(detail::policy_for<Out>(), first, last, result, old_value, new_value);
}
template <typename It, typename Pred, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void replace_if(It first, It last, Pred pred, const T& new_value) {
  thrust::replace_if(detail::policy_for<It>(), first, last, pred, new_value);
}
template <typename It, typename St, typename Pred, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void replace_if(It first, It last, St stencil, Pred pred, const T& new_value) {
  thrust::replace_if(detail::policy_for<It>(), first, last, stencil, pred, new_value);
}
template <typename It, typename T, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void replace(It first, It last, const T& old_value, const T& new_value) {
  thrust::replace(detail::policy_for<It>(), first, last, old_value, new_value);
}

}  // namespace thrust
