// thrust::allocate_unique and its relatives: one object, or n, from an allocator, owned by a
// std::unique_ptr whose deleter gives the storage back to that allocator
// (thrust/allocate_unique.h:70-440; testing/universal_memory.cu:35-110).
//
// What get() returns is the allocator's pointer; a device_ptr is read through it (`*p.get()`, `p->member`),
// not through std::unique_ptr's own operator*, which wants a plain reference.
//
// Storage behind a plain pointer is constructed in place.  Storage behind a device_ptr (device or
// universal memory) receives the bytes of an object built on the host, and is released without a
// destructor call: T must be trivially copyable and trivially destructible there, which is what
// device_new / device_delete ask for as well.
#pragma once
#include <cstddef>
#include <memory>
#include <new>
#include <type_traits>
#include <utility>

#include <thrust/device_ptr.h>
#include <thrust/uninitialized_fill.h>

namespace thrust {
namespace detail {
template <typename T, typename... Args>
inline void construct_at(T* p, Args&&... args) { ::new (static_cast<void*>(p)) T(std::forward<Args>(args)...); }
template <typename T, typename... Args>
inline void construct_at(thrust::device_ptr<T> p, Args&&... args) {
  static_assert(std::is_trivially_copyable<T>::value, "objects in device memory are written as their bytes");
  const T built(std::forward<Args>(args)...);
  thrust::system::hip::detail::throw_on_error(thrust_amd_memcpy(p.get(), &built, sizeof(T), THRUST_AMD_H2D, nullptr),
                                              "allocate_unique: construct");
}
template <typename T>
inline void destroy_n(T* p, std::size_t n) {
  for (std::size_t i = 0; i < n; ++i) p[i].~T();
}
template <typename T>
inline void destroy_n(thrust::device_ptr<T>, std::size_t) {
  static_assert(std::is_trivially_destructible<T>::value, "objects in device memory are released without a destructor call");
}
template <typename T, typename V>
inline void fill_n_new(T* p, std::size_t n, const V& v) {
  for (std::size_t i = 0; i < n; ++i) construct_at(p + i, v);
}
template <typename T, typename V>
inline void fill_n_new(thrust::device_ptr<T> p, std::size_t n, const V& v) { thrust::uninitialized_fill_n(p, n, T(v)); }

template <typename Alloc, typename T>
struct rebound_allocator { typedef typename std::allocator_traits<Alloc>::template rebind_alloc<T> type; };
}  // namespace detail

// Destroys (unless Uninitialized) and deallocates one T.
template <typename T, typename Allocator, bool Uninitialized = false>
struct allocator_delete final {
  typedef typename detail::rebound_allocator<Allocator, T>::type allocator_type;
  typedef typename std::allocator_traits<allocator_type>::pointer pointer;
  template <typename A>
  allocator_delete(A&& a) : alloc_(std::forward<A>(a)) {}
  void operator()(pointer p) {
    if (!Uninitialized) detail::destroy_n(p, 1);
    alloc_.deallocate(p, 1);
  }
  allocator_type& get_allocator() noexcept { return alloc_; }

 private:
  allocator_type alloc_;
};
template <typename T, typename Allocator>
using uninitialized_allocator_delete = allocator_delete<T, Allocator, true>;

// Destroys (unless Uninitialized) and deallocates the n objects it was made for.
template <typename T, typename Allocator, bool Uninitialized = false>
struct array_allocator_delete final {
  typedef typename detail::rebound_allocator<Allocator, T>::type allocator_type;
  typedef typename std::allocator_traits<allocator_type>::pointer pointer;
  template <typename A>
  array_allocator_delete(A&& a, std::size_t n) : alloc_(std::forward<A>(a)), count_(n) {}
  void operator()(pointer p) {
    if (!Uninitialized) detail::destroy_n(p, count_);
    alloc_.deallocate(p, count_);
  }
  allocator_type& get_allocator() noexcept { return alloc_; }
  std::size_t size() const noexcept { return count_; }

 private:
  allocator_type alloc_;
  std::size_t count_;
};
template <typename T, typename Allocator>
using uninitialized_array_allocator_delete = array_allocator_delete<T, Allocator, true>;

template <typename T, typename Allocator, typename... Args>
inline std::unique_ptr<T, allocator_delete<T, Allocator> > allocate_unique(const Allocator& alloc, Args&&... args) {
  typename detail::rebound_allocator<Allocator, T>::type a(alloc);
  auto p = a.allocate(1);
  try {
    detail::construct_at(p, std::forward<Args>(args)...);
  } catch (...) {
    a.deallocate(p, 1);
    throw;
  }
  return std::unique_ptr<T, allocator_delete<T, Allocator> >(p, allocator_delete<T, Allocator>(a));
}
template <typename T, typename Allocator>
inline std::unique_ptr<T, uninitialized_allocator_delete<T, Allocator> > uninitialized_allocate_unique(const Allocator& alloc) {
  typename detail::rebound_allocator<Allocator, T>::type a(alloc);
  auto p = a.allocate(1);
  return std::unique_ptr<T, uninitialized_allocator_delete<T, Allocator> >(p, uninitialized_allocator_delete<T, Allocator>(a));
}
// n copies of T(args...)
template <typename T, typename Allocator, typename Size, typename... Args>
inline std::unique_ptr<T[], array_allocator_delete<T, Allocator> > allocate_unique_n(const Allocator& alloc, Size n,
                                                                                    Args&&... args) {
  typename detail::rebound_allocator<Allocator, T>::type a(alloc);
  auto p = a.allocate((std::size_t)n);
  try {
    detail::fill_n_new(p, (std::size_t)n, T(std::forward<Args>(args)...));
  } catch (...) {
    a.deallocate(p, (std::size_t)n);
    throw;
  }
  return std::unique_ptr<T[], array_allocator_delete<T, Allocator> >(p, array_allocator_delete<T, Allocator>(a, (std::size_t)n));
}
template <typename T, typename Allocator, typename Size>
inline std::unique_ptr<T[], uninitialized_array_allocator_delete<T, Allocator> > uninitialized_allocate_unique_n(
    const Allocator& alloc, Size n) {
  typename detail::rebound_allocator<Allocator, T>::type a(alloc);
  auto p = a.allocate((std::size_t)n);
  return std::unique_ptr<T[], uninitialized_array_allocator_delete<T, Allocator> >(
      p, uninitialized_array_allocator_delete<T, Allocator>(a, (std::size_t)n));
}
}  // namespace thrust
