// thrust::device_malloc_allocator: an allocator over device_malloc / device_free
// (thrust/device_malloc_allocator.h:50-180).
#pragma once
#include <cstddef>
#include <limits>
#include <new>

#include <thrust/device_ptr.h>
#include <thrust/device_reference.h>

namespace thrust {

template <typename T>
class device_malloc_allocator {
 public:
  typedef T value_type;
  typedef device_ptr<T> pointer;
  typedef device_ptr<const T> const_pointer;
  typedef device_reference<T> reference;
  typedef device_reference<const T> const_reference;
  typedef std::size_t size_type;
  typedef std::ptrdiff_t difference_type;
  template <typename U>
  struct rebind { typedef device_malloc_allocator<U> other; };

  device_malloc_allocator() {}
  template <typename U>
  device_malloc_allocator(const device_malloc_allocator<U>&) {}
  pointer address(reference r) { return &r; }
  pointer allocate(size_type n, const void* = nullptr) {
    if (n > max_size()) throw std::bad_alloc();
    return thrust::device_malloc<T>(n);
  }
  void deallocate(pointer p, size_type) { thrust::device_free(p); }
  size_type max_size() const { return (std::numeric_limits<size_type>::max)() / sizeof(T); }
  bool operator==(const device_malloc_allocator&) const { return true; }
  bool operator!=(const device_malloc_allocator& other) const { return !(*this == other); }
};

}  // namespace thrust
