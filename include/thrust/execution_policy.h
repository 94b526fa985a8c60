// thrust::host, thrust::device, thrust::seq, thrust::hip::par, par.on(stream), par(alloc),
// par(alloc).on(stream).
#pragma once
#include <cstddef>
#include <utility>

#include <thrust/detail/execution_policy.h>

namespace thrust {
namespace detail {
struct host_t : thrust::host_execution_policy<host_t> {};
struct seq_t : thrust::system::cpp::execution_policy<seq_t> {};
}  // namespace detail

static const detail::host_t host;
static const detail::seq_t seq;

namespace system {
namespace hip {

struct after_policy;  // thrust/future.h: a policy with dependencies, for the asynchronous algorithms

// Policy bound to a stream: thrust::hip::par.on(stream).
struct stream_policy : execution_policy<stream_policy> {
  void* stream;
  explicit stream_policy(void* s) : stream(s) {}
  template <typename... Events>
  after_policy after(const Events&... events) const;  // defined in thrust/future.h
};
inline void* get_stream(const stream_policy& p) { return p.stream; }

// Policy carrying a user allocator for temporary storage: thrust::hip::par(alloc), optionally
// .on(stream).  Every algorithm then takes its scratch memory from alloc.allocate(n) (n in
// units of Alloc::value_type; the result may be a raw device pointer or a device_ptr) and
// returns it with alloc.deallocate(p, n) before it returns -- the contract of the
// reference's examples/cuda/custom_temporary_allocation.cu:44-140.  The allocator is held
// by reference and must outlive the call.
template <typename Alloc>
struct allocator_policy : execution_policy<allocator_policy<Alloc> > {
  Alloc* alloc;
  void* stream;
  explicit allocator_policy(Alloc& a, void* s = nullptr) : alloc(&a), stream(s) {}
  allocator_policy on(void* s) const { return allocator_policy(*alloc, s); }
};
template <typename Alloc>
inline void* get_stream(const allocator_policy<Alloc>& p) { return p.stream; }

namespace detail {
template <typename Alloc>
struct allocator_thunks {
  typedef typename Alloc::value_type value_type;
  typedef decltype(std::declval<Alloc&>().allocate(std::size_t())) pointer;
  static std::size_t count(std::size_t bytes) { return (bytes + sizeof(value_type) - 1) / sizeof(value_type); }
  static value_type* to_raw(value_type* p) { return p; }
  template <typename P>
  static value_type* to_raw(const P& p) { return p.get(); }
  static void* acquire(void* ctx, std::size_t bytes) {
    return to_raw(static_cast<Alloc*>(ctx)->allocate(count(bytes)));
  }
  static void release(void* ctx, void* p, std::size_t bytes) {
    static_cast<Alloc*>(ctx)->deallocate(pointer(static_cast<value_type*>(p)), count(bytes));
  }
};
}  // namespace detail
template <typename Alloc>
inline detail::temp_source get_temp_source(const allocator_policy<Alloc>& p) {
  return detail::temp_source{p.alloc, &detail::allocator_thunks<Alloc>::acquire,
                             &detail::allocator_thunks<Alloc>::release};
}

// Policy carrying a memory resource for temporary storage: thrust::hip::par(&resource) with
// resource a thrust::mr::memory_resource whose pointer is void* (device-accessible) or
// device_ptr<void> (the reference accepts a resource pointer in the same place,
// thrust/detail/allocator_aware_execution_policy.h:60-90).
template <typename Resource>
struct resource_policy : execution_policy<resource_policy<Resource> > {
  Resource* resource;
  void* stream;
  explicit resource_policy(Resource* r, void* s = nullptr) : resource(r), stream(s) {}
  resource_policy on(void* s) const { return resource_policy(resource, s); }
};
template <typename Resource>
inline void* get_stream(const resource_policy<Resource>& p) { return p.stream; }
namespace detail {
template <typename Resource>
struct resource_thunks {
  static void* to_raw(void* p) { return p; }
  template <typename P>
  static void* to_raw(const P& p) { return p.get(); }
  static void* acquire(void* ctx, std::size_t bytes) { return to_raw(static_cast<Resource*>(ctx)->allocate(bytes, 256)); }
  static void release(void* ctx, void* p, std::size_t bytes) {
    static_cast<Resource*>(ctx)->deallocate(typename Resource::pointer(p), bytes, 256);
  }
};
}  // namespace detail
template <typename Resource>
inline detail::temp_source get_temp_source(const resource_policy<Resource>& p) {
  return detail::temp_source{p.resource, &detail::resource_thunks<Resource>::acquire,
                             &detail::resource_thunks<Resource>::release};
}

struct par_t : execution_policy<par_t> {
  // `stream` is a hipStream_t; it is taken as void* so that user code needs no HIP headers.
  stream_policy on(void* stream) const { return stream_policy(stream); }
  template <typename Alloc>
  allocator_policy<Alloc> operator()(Alloc& alloc) const { return allocator_policy<Alloc>(alloc); }
  template <typename Resource>
  resource_policy<Resource> operator()(Resource* resource) const { return resource_policy<Resource>(resource); }
  template <typename... Events>
  after_policy after(const Events&... events) const;  // defined in thrust/future.h
};
static const par_t par;

namespace detail {
// The stream of any policy of this system: the most derived get_stream wins.
template <typename Derived>
inline void* stream_of(execution_policy<Derived>& p) {
  return get_stream(thrust::detail::derived_cast(p));
}
template <typename Derived>
inline temp_source temp_source_of(execution_policy<Derived>& p) {
  return get_temp_source(thrust::detail::derived_cast(p));
}
}  // namespace detail

}  // namespace hip
}  // namespace system

namespace detail {
// thrust::device: the device system's default policy, with the same builders as hip::par.
struct device_t : thrust::device_execution_policy<device_t> {
  system::hip::stream_policy on(void* stream) const { return system::hip::stream_policy(stream); }
  template <typename Alloc>
  system::hip::allocator_policy<Alloc> operator()(Alloc& alloc) const { return system::hip::allocator_policy<Alloc>(alloc); }
  template <typename Resource>
  system::hip::resource_policy<Resource> operator()(Resource* resource) const {
    return system::hip::resource_policy<Resource>(resource);
  }
  template <typename... Events>
  system::hip::after_policy after(const Events&... events) const;  // defined in thrust/future.h
};
}  // namespace detail
static const detail::device_t device;

namespace hip = system::hip;
namespace cpp {
using thrust::system::cpp::execution_policy;
using thrust::system::cpp::tag;
static const thrust::detail::seq_t par;
}  // namespace cpp

}  // namespace thrust
