// thrust::retag / thrust::reinterpret_tag: the same iterator under another system's tag
// (thrust/iterator/retag.h:30-60).  Systems here are told apart by iterator type (device_ptr against
// plain pointers) or by the policy argument, so the forms the two systems need are:
// a pointer or device_ptr seen as the device system's, and a device_ptr seen as the host system's
// (meaningful only for storage that the host can address, such as universal_vector's).
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/execution_policy.h>

namespace thrust {
namespace detail {
template <typename Tag, typename T, bool HOST = std::is_convertible<Tag, thrust::host_system_tag>::value>
struct retagged { typedef thrust::device_ptr<T> type; };
template <typename Tag, typename T>
struct retagged<Tag, T, true> { typedef T* type; };
}  // namespace detail
template <typename Tag, typename T>
inline typename detail::retagged<Tag, T>::type reinterpret_tag(T* p) { return typename detail::retagged<Tag, T>::type(p); }
template <typename Tag, typename T>
inline typename detail::retagged<Tag, T>::type reinterpret_tag(const thrust::device_ptr<T>& p) {
  return typename detail::retagged<Tag, T>::type(p.get());
}
template <typename Tag, typename T>
inline typename detail::retagged<Tag, T>::type retag(T* p) { return reinterpret_tag<Tag>(p); }
template <typename Tag, typename T>
inline typename detail::retagged<Tag, T>::type retag(const thrust::device_ptr<T>& p) { return reinterpret_tag<Tag>(p); }
}  // namespace thrust
