// thrust::mr::allocator<T, MR> and thrust::mr::stateless_resource_allocator<T, MR>:
// allocators (the interface containers use) over a memory resource
// (thrust/mr/allocator.h:44-250 of the reference).  allocate(n) returns MR's pointer type
// rebound to T: T* for void*, device_ptr<T> for device_ptr<void>.
#pragma once
#include <cstddef>
#include <new>
#include <type_traits>

#include <thrust/mr/memory_resource.h>
#include <thrust/mr/polymorphic_adaptor.h>

namespace thrust {
template <typename T> class device_ptr;

namespace mr {
namespace detail {
template <typename Pointer, typename T> struct rebind_pointer;
template <typename U, typename T> struct rebind_pointer<U*, T> {
  typedef T* type;
  static type cast(U* p) { return static_cast<T*>(static_cast<void*>(p)); }
  static U* back(T* p) { return static_cast<U*>(static_cast<void*>(p)); }
};
template <typename U, typename T> struct rebind_pointer<thrust::device_ptr<U>, T> {
  typedef thrust::device_ptr<T> type;
  static type cast(const thrust::device_ptr<U>& p) { return type(static_cast<T*>(static_cast<void*>(p.get()))); }
  static thrust::device_ptr<U> back(const type& p) {
    return thrust::device_ptr<U>(static_cast<U*>(static_cast<void*>(const_cast<typename std::remove_const<T>::type*>(p.get()))));
  }
};
}  // namespace detail

template <typename T, typename MR>
class allocator {
 public:
  typedef T value_type;
  typedef typename detail::rebind_pointer<typename MR::pointer, T>::type pointer;
  typedef std::size_t size_type;
  template <typename U> struct rebind { typedef allocator<U, MR> other; };

  explicit allocator(MR* resource) : resource_(resource) {}
  template <typename U>
  allocator(const allocator<U, MR>& other) : resource_(other.resource()) {}

  pointer allocate(size_type n) {
    if (n > (~size_type(0)) / sizeof(T)) throw std::bad_alloc();
    return detail::rebind_pointer<typename MR::pointer, T>::cast(resource_->allocate(n * sizeof(T), alignof(T)));
  }
  void deallocate(pointer p, size_type n) {
    resource_->deallocate(detail::rebind_pointer<typename MR::pointer, T>::back(p), n * sizeof(T), alignof(T));
  }
  MR* resource() const { return resource_; }

 private:
  MR* resource_;
};
template <typename T, typename MR>
inline bool operator==(const allocator<T, MR>& a, const allocator<T, MR>& b) { return *a.resource() == *b.resource(); }
template <typename T, typename MR>
inline bool operator!=(const allocator<T, MR>& a, const allocator<T, MR>& b) { return !(a == b); }

// Uses the one global instance of MR.
template <typename T, typename MR>
class stateless_resource_allocator : public allocator<T, MR> {
 public:
  template <typename U> struct rebind { typedef stateless_resource_allocator<U, MR> other; };
  stateless_resource_allocator() : allocator<T, MR>(get_global_resource<MR>()) {}
  template <typename U>
  stateless_resource_allocator(const stateless_resource_allocator<U, MR>&) : allocator<T, MR>(get_global_resource<MR>()) {}
};

// An allocator over whichever resource is behind a polymorphic_adaptor_resource
// (thrust/mr/allocator.h:215-240).
template <typename T, typename Pointer = void*>
class polymorphic_allocator : public allocator<T, polymorphic_adaptor_resource<Pointer> > {
 public:
  template <typename U> struct rebind { typedef polymorphic_allocator<U, Pointer> other; };
  polymorphic_allocator(polymorphic_adaptor_resource<Pointer>* resource)
      : allocator<T, polymorphic_adaptor_resource<Pointer> >(resource) {}
  template <typename U>
  polymorphic_allocator(const polymorphic_allocator<U, Pointer>& o)
      : allocator<T, polymorphic_adaptor_resource<Pointer> >(o.resource()) {}
};

}  // namespace mr
}  // namespace thrust
