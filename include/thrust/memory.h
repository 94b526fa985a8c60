// thrust/memory.h: raw_pointer_cast, raw_reference_cast, and storage by system tag:
// thrust::malloc / thrust::free and get_temporary_buffer / return_temporary_buffer
// (thrust/memory.h:200-390; testing/memory.cu, get_temporary_buffer examples in the header).
#pragma once
#include <cstddef>
#include <cstdlib>

#include <thrust/detail/raw_reference_cast.h>
#include <thrust/device_free.h>
#include <thrust/device_malloc.h>
#include <thrust/device_ptr.h>
#include <thrust/execution_policy.h>
#include <thrust/pair.h>

namespace thrust {
// The pointer type of a system: plain for the host system, device_ptr for the device system
// (thrust/memory.h:60-190 declares it as a class of its own; here the two systems' pointer
// types are named through it).
template <typename T, typename Tag>
using pointer = typename std::conditional<std::is_convertible<Tag, thrust::host_system_tag>::value, T*,
                                          thrust::device_ptr<T> >::type;

namespace system {
namespace cpp {
template <typename D>
inline void* raw_malloc(execution_policy<D>&, std::size_t bytes) { return std::malloc(bytes); }
template <typename T, typename D>
inline T* raw_malloc(execution_policy<D>&, std::size_t n, T*) { return static_cast<T*>(std::malloc(n * sizeof(T))); }
template <typename D, typename P>
inline void raw_free(execution_policy<D>&, P p) { std::free(const_cast<void*>(static_cast<const void*>(p))); }
}  // namespace cpp
namespace hip {
template <typename D>
inline thrust::device_ptr<void> raw_malloc(execution_policy<D>&, std::size_t bytes) { return thrust::device_malloc(bytes); }
template <typename T, typename D>
inline thrust::device_ptr<T> raw_malloc(execution_policy<D>&, std::size_t n, T*) { return thrust::device_malloc<T>(n); }
template <typename D, typename T>
inline void raw_free(execution_policy<D>&, thrust::device_ptr<T> p) { thrust::device_free(p); }
template <typename D, typename T>
inline void raw_free(execution_policy<D>&, T* p) { thrust::device_free(thrust::device_ptr<T>(p)); }
}  // namespace hip
}  // namespace system

// n bytes (or n objects of T, uninitialised) in the memory of exec's system.
// (each system answers under the names raw_malloc / raw_free, found through its tag; the typed
// form takes a null T* to say which T)
template <typename D>
inline auto malloc(const detail::execution_policy_base<D>& exec, std::size_t bytes)
    -> decltype(raw_malloc(detail::derived_cast(detail::strip_const(exec)), bytes)) {
  return raw_malloc(detail::derived_cast(detail::strip_const(exec)), bytes);
}
template <typename T, typename D>
inline auto malloc(const detail::execution_policy_base<D>& exec, std::size_t n)
    -> decltype(raw_malloc(detail::derived_cast(detail::strip_const(exec)), n, static_cast<T*>(nullptr))) {
  return raw_malloc(detail::derived_cast(detail::strip_const(exec)), n, static_cast<T*>(nullptr));
}
template <typename D, typename Pointer>
inline void free(const detail::execution_policy_base<D>& exec, Pointer p) {
  raw_free(detail::derived_cast(detail::strip_const(exec)), p);
}

// Room for up to n objects of T and how many it holds; given back with
// return_temporary_buffer (thrust/memory.h:300-390).
template <typename T, typename D>
inline auto get_temporary_buffer(const detail::execution_policy_base<D>& exec, std::ptrdiff_t n)
    -> thrust::pair<decltype(thrust::malloc<T>(exec, (std::size_t)n)), std::ptrdiff_t> {
  typedef decltype(thrust::malloc<T>(exec, (std::size_t)n)) pointer;
  pointer p = thrust::malloc<T>(exec, (std::size_t)n);
  return thrust::pair<pointer, std::ptrdiff_t>(p, raw_pointer_cast(p) ? n : 0);
}
template <typename D, typename Pointer>
inline void return_temporary_buffer(const detail::execution_policy_base<D>& exec, Pointer p, std::ptrdiff_t = 0) {
  thrust::free(exec, p);
}
}  // namespace thrust
