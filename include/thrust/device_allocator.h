// thrust::device_memory_resource and thrust::device_allocator<T>.
//
// device_memory_resource hands out device memory from the device system's malloc / free
// (thrust/system/cuda/memory_resource.h:40-110 and thrust/device_allocator.h:40-140 of the
// reference); its pointer type is device_ptr<void>.  device_allocator<T> is the stateless
// allocator over it and the default allocator of device_vector.
#pragma once
#include <cstddef>

#include <thrust/device_ptr.h>
#include <thrust/mr/allocator.h>
#include <thrust/mr/memory_resource.h>

namespace thrust {
namespace system {
namespace hip {
class memory_resource : public thrust::mr::memory_resource<thrust::device_ptr<void> > {
 protected:
  thrust::device_ptr<void> do_allocate(std::size_t bytes, std::size_t) override { return thrust::device_malloc(bytes); }
  void do_deallocate(thrust::device_ptr<void> p, std::size_t, std::size_t) override {
    thrust::system::hip::detail::throw_on_error(thrust_amd_free(p.get()), "device_memory_resource: free");
  }
  bool do_is_equal(const thrust::mr::memory_resource<thrust::device_ptr<void> >& other) const noexcept override {
    return dynamic_cast<const memory_resource*>(&other) != nullptr;
  }
};
}  // namespace hip
}  // namespace system

typedef system::hip::memory_resource device_memory_resource;

// A resource whose pointers are device_ptr over one whose pointers are the system's own
// (thrust/device_allocator.h:46-95).  The device system's pointers are device_ptr already, so
// this forwards.
template <typename Upstream>
class device_ptr_memory_resource final : public thrust::mr::memory_resource<thrust::device_ptr<void> > {
 public:
  device_ptr_memory_resource() : upstream_(thrust::mr::get_global_resource<Upstream>()) {}
  device_ptr_memory_resource(Upstream* upstream) : upstream_(upstream) {}

 protected:
  thrust::device_ptr<void> do_allocate(std::size_t bytes, std::size_t alignment) override {
    return thrust::device_ptr<void>(raw_pointer_cast(upstream_->allocate(bytes, alignment)));
  }
  void do_deallocate(thrust::device_ptr<void> p, std::size_t bytes, std::size_t alignment) override {
    upstream_->deallocate(typename Upstream::pointer(p.get()), bytes, alignment);
  }

 private:
  Upstream* upstream_;
};

template <typename T>
class device_allocator : public thrust::mr::stateless_resource_allocator<T, device_memory_resource> {
 public:
  template <typename U> struct rebind { typedef device_allocator<U> other; };
  device_allocator() {}
  template <typename U>
  device_allocator(const device_allocator<U>&) {}
};

}  // namespace thrust
