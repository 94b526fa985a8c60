// thrust::universal_vector, thrust::universal_allocator, thrust::universal_memory_resource.
//
// A vector whose storage host code and kernels both address (thrust/universal_vector.h,
// thrust/universal_allocator.h of the reference).  Its iterators are device_ptr, so
// algorithms run on the device system; host code may also go straight through
// thrust::raw_pointer_cast(v.data()) once the work that wrote the vector has been
// synchronised (the blocking algorithms have, when they return).
#pragma once
#include <thrust/device_allocator.h>
#include <thrust/device_vector.h>

namespace thrust {
namespace system {
namespace hip {
class universal_memory_resource : public thrust::mr::memory_resource<thrust::device_ptr<void> > {
 protected:
  thrust::device_ptr<void> do_allocate(std::size_t bytes, std::size_t) override {
    void* p = nullptr;
    const int rc = thrust_amd_malloc_universal(&p, bytes);
    if (rc != 0) throw thrust::system::detail::bad_alloc(thrust_amd_error_string(rc));
    return thrust::device_ptr<void>(p);
  }
  void do_deallocate(thrust::device_ptr<void> p, std::size_t, std::size_t) override {
    thrust::system::hip::detail::throw_on_error(thrust_amd_free_universal(p.get()), "universal_memory_resource: free");
  }
  bool do_is_equal(const thrust::mr::memory_resource<thrust::device_ptr<void> >& other) const noexcept override {
    return dynamic_cast<const universal_memory_resource*>(&other) != nullptr;
  }
};
}  // namespace hip
}  // namespace system

typedef system::hip::universal_memory_resource universal_memory_resource;

template <typename T>
class universal_allocator : public thrust::mr::stateless_resource_allocator<T, universal_memory_resource> {
 public:
  template <typename U> struct rebind { typedef universal_allocator<U> other; };
  universal_allocator() {}
  template <typename U>
  universal_allocator(const universal_allocator<U>&) {}
};

template <typename T, typename Alloc = universal_allocator<T> >
using universal_vector = device_vector<T, Alloc>;

}  // namespace thrust
