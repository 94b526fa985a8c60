// thrust::mr::memory_resource: the polymorphic interface memory is obtained through.
//
// allocate(bytes, alignment) / deallocate(pointer, bytes, alignment) forward to the virtual
// do_allocate / do_deallocate of the concrete resource; two resources compare equal when
// memory taken from one may be returned to the other (thrust/mr/memory_resource.h:41-120 of
// the reference, modelled on std::pmr).  Pointer is void* for host memory and
// thrust::device_ptr<void> for the device system's resources.
#pragma once
#include <cstddef>

namespace thrust {
namespace mr {

template <typename Pointer = void*>
class memory_resource {
 public:
  typedef Pointer pointer;
  virtual ~memory_resource() {}
  pointer allocate(std::size_t bytes, std::size_t alignment = alignof(std::max_align_t)) {
    return do_allocate(bytes, alignment);
  }
  void deallocate(pointer p, std::size_t bytes, std::size_t alignment = alignof(std::max_align_t)) {
    do_deallocate(p, bytes, alignment);
  }
  bool is_equal(const memory_resource& other) const noexcept { return do_is_equal(other); }

 protected:
  virtual pointer do_allocate(std::size_t bytes, std::size_t alignment) = 0;
  virtual void do_deallocate(pointer p, std::size_t bytes, std::size_t alignment) = 0;
  virtual bool do_is_equal(const memory_resource& other) const noexcept { return this == &other; }
};

template <typename Pointer>
inline bool operator==(const memory_resource<Pointer>& a, const memory_resource<Pointer>& b) noexcept {
  return &a == &b || a.is_equal(b);
}
template <typename Pointer>
inline bool operator!=(const memory_resource<Pointer>& a, const memory_resource<Pointer>& b) noexcept {
  return !(a == b);
}

// One instance per resource type for the stateless allocators (thrust/mr/memory_resource.h:170-200).
template <typename MR>
inline MR* get_global_resource() {
  static MR resource;
  return &resource;
}

}  // namespace mr
}  // namespace thrust
