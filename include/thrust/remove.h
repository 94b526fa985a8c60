// thrust::remove, remove_if, remove_copy and remove_copy_if.
//
// Stable removal of the elements that equal a value or satisfy a predicate (of the element
// or of a stencil element); the in-place forms return the new logical end.  The reference's
// device system runs copy_if with the negated predicate, in place for remove / remove_if
// (thrust/system/cuda/detail/remove.h:40-131); the host system is the sequential loop
// (thrust/system/detail/sequential/remove.h:41-140).  On the device system the predicate
// must be one of the recognised forms listed in thrust/functional.h.
#pragma once
#include <thrust/copy.h>
#include <thrust/functional.h>
#include <thrust/system/hip/detail/backend.h>

namespace thrust {

template <typename D, typename In, typename Out, typename Pred>
Out remove_copy_if(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Pred pred);
template <typename D, typename In, typename St, typename Out, typename Pred>
Out remove_copy_if(const detail::execution_policy_base<D>& exec, In first, In last, St stencil, Out result, Pred pred);
template <typename D, typename It, typename Pred>
It remove_if(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred);
template <typename D, typename It, typename St, typename Pred>
It remove_if(const detail::execution_policy_base<D>& exec, It first, It last, St stencil, Pred pred);

namespace system {
namespace detail {
namespace generic {
// remove(value) = remove_if(x == value), compared in the element type
// (thrust/system/detail/generic/remove.inl:44-72)
template <typename D, typename It, typename T>
It remove(thrust::execution_policy<D>& exec, It first, It last, const T& value) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  using namespace thrust::placeholders;
  return thrust::remove_if(exec, first, last, _1 == static_cast<V>(value));
}
template <typename D, typename In, typename Out, typename T>
Out remove_copy(thrust::execution_policy<D>& exec, In first, In last, Out result, const T& value) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  using namespace thrust::placeholders;
  return thrust::remove_copy_if(exec, first, last, result, _1 == static_cast<V>(value));
}
}  // namespace generic
}  // namespace detail

namespace cpp {
template <typename D, typename In, typename St, typename Out, typename Pred>
Out remove_copy_if(execution_policy<D>&, In first, In last, St stencil, Out result, Pred pred) {
  for (; first != last; ++first, ++stencil)
    if (!pred(*stencil)) { *result = *first; ++result; }
  return result;
}
template <typename D, typename In, typename Out, typename Pred>
Out remove_copy_if(execution_policy<D>& exec, In first, In last, Out result, Pred pred) {
  return remove_copy_if(exec, first, last, first, result, pred);
}
template <typename D, typename It, typename St, typename Pred>
It remove_if(execution_policy<D>& exec, It first, It last, St stencil, Pred pred) {
  return remove_copy_if(exec, first, last, stencil, first, pred);  // writes never pass the read position
}
template <typename D, typename It, typename Pred>
It remove_if(execution_policy<D>& exec, It first, It last, Pred pred) {
  return remove_copy_if(exec, first, last, first, first, pred);
}
}  // namespace cpp

namespace hip {
template <typename D, typename In, typename Out, typename Pred>
Out remove_copy_if(execution_policy<D>& exec, In first, In last, Out result, Pred pred) {
  return detail::copy_if_any(exec, first, last, first, std::false_type(), result, pred, true);
}
template <typename D, typename In, typename St, typename Out, typename Pred>
Out remove_copy_if(execution_policy<D>& exec, In first, In last, St stencil, Out result, Pred pred) {
  return detail::copy_if_any(exec, first, last, stencil, std::true_type(), result, pred, true);
}
// in place: the compaction kernel writes a tile only after every earlier tile has been read
template <typename D, typename It, typename Pred>
It remove_if(execution_policy<D>& exec, It first, It last, Pred pred) {
  return remove_copy_if(exec, first, last, first, pred);
}
template <typename D, typename It, typename St, typename Pred>
It remove_if(execution_policy<D>& exec, It first, It last, St stencil, Pred pred) {
  return remove_copy_if(exec, first, last, stencil, first, pred);
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry points
template <typename D, typename In, typename Out, typename Pred>
Out remove_copy_if(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Pred pred) {
  return remove_copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, result, pred);
}
template <typename D, typename In, typename St, typename Out, typename Pred>
Out remove_copy_if(const detail::execution_policy_base<D>& exec, In first, In last, St stencil, Out result, Pred pred) {
  return remove_copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, result, pred);
}
template <typename D, typename It, typename Pred>
It remove_if(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return remove_if(detail::derived_cast(detail::strip_const(exec)), first, last, pred);
}
template <typename D, typename It, typename St, typename Pred>
It remove_if(const detail::execution_policy_base<D>& exec, It first, It last, St stencil, Pred pred) {
  return remove_if(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, pred);
}
template <typename D, typename It, typename T>
It remove(const detail::execution_policy_base<D>& exec, It first, It last, const T& value) {
  using thrust::system::detail::generic::remove;
  return remove(detail::derived_cast(detail::strip_const(exec)), first, last, value);
}
template <typename D, typename In, typename Out, typename T>
Out remove_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result, const T& value) {
  using thrust::system::detail::generic::remove_copy;
  return remove_copy(detail::derived_cast(detail::strip_const(exec)), first, last, result, value);
}

// without a policy
template <typename In, typename Out, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out remove_copy_if(In first, In last, Out result, Pred pred) {
  return thrust::remove_copy_if(detail::policy_for<In>(), first, last, result, pred);
}
template <typename In, typename St, typename Out, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out remove_copy_if(In first, In last, St stencil, Out result, Pred pred) {
  return thrust::remove_copy_if(detail::policy_for<In>(), first, last, stencil, result, pred);
}
template <typename It, typename Pred>
It remove_if(It first, It last, Pred pred) {
  return thrust::remove_if(detail::policy_for<It>(), first, last, pred);
}
template <typename It, typename St, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It remove_if(It first, It last, St stencil, Pred pred) {
  return thrust::remove_if(detail::policy_for<It>(), first, last, stencil, pred);
}
template <typename It, typename T>
It remove(It first, It last, const T& value) {
  return thrust::remove(detail::policy_for<It>(), first, last, value);
}
template <typename In, typename Out, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out remove_copy(In first, In last, Out result, const T& value) {
  return thrust::remove_copy(detail::policy_for<In>(), first, last, result, value);
}

}  // namespace thrust
