// Execution-policy plumbing: CRTP bases, derived_cast, the system tags.
//
// Dispatch works as in the reference (thrust/detail/execution_policy.h:30-80): a public
// entry point takes `const execution_policy_base<Derived>&`, casts to the derived policy
// and makes an UNQUALIFIED call, so that argument-dependent lookup finds
//   - a user's overload for a policy derived from device_execution_policy (interception,
//     as in the reference's examples/minimal_custom_backend.cu:17-37), else
//   - the system's overload taking hip::execution_policy<Derived>& or
//     cpp::execution_policy<Derived>&, a nearer base than execution_policy_base.
#pragma once
#include <cstddef>

#include <thrust/detail/config.h>

namespace thrust {
namespace detail {

struct execution_policy_marker {};

template <typename Derived>
struct execution_policy_base : execution_policy_marker {};

template <typename Derived>
constexpr execution_policy_base<Derived>& strip_const(const execution_policy_base<Derived>& x) {
  return const_cast<execution_policy_base<Derived>&>(x);
}
template <typename Derived>
constexpr Derived& derived_cast(execution_policy_base<Derived>& x) {
  return static_cast<Derived&>(x);
}
template <typename Derived>
constexpr const Derived& derived_cast(const execution_policy_base<Derived>& x) {
  return static_cast<const Derived&>(x);
}

}  // namespace detail

template <typename Derived>
struct execution_policy : thrust::detail::execution_policy_base<Derived> {};

namespace system {
namespace cpp {
// Sequential host system.
template <typename Derived>
struct execution_policy : thrust::execution_policy<Derived> {};
struct tag : execution_policy<tag> {};
}  // namespace cpp
namespace hip {
// The gfx950 device system.  get_stream(policy) yields the hipStream_t (as void*) the
// algorithms enqueue on; the default is the null stream, `par.on(s)` carries another one
// (the reference: cuda_cub::stream(policy), thrust/system/cuda/detail/util.h:44-68 and
// par.on(), thrust/system/cuda/detail/par.h:46-108).
template <typename Derived>
struct execution_policy : thrust::execution_policy<Derived> {};
struct tag : execution_policy<tag> {};
template <typename Derived>
inline void* get_stream(const execution_policy<Derived>&) { return nullptr; }

// get_temp_source(policy) says where an algorithm's temporary storage comes from: the
// library's arena (all members null, the default) or an allocator the caller attached
// with par(alloc) (the reference: thrust/detail/allocator_aware_execution_policy.h:37-100
// and temporary_array, thrust/detail/temporary_array.h).
namespace detail {
struct temp_source {
  void* ctx;
  void* (*acquire)(void* ctx, std::size_t bytes);
  void (*release)(void* ctx, void* p, std::size_t bytes);
};
}  // namespace detail
template <typename Derived>
inline detail::temp_source get_temp_source(const execution_policy<Derived>&) {
  return detail::temp_source{nullptr, nullptr, nullptr};
}
}  // namespace hip
}  // namespace system

template <typename Derived>
struct host_execution_policy : thrust::system::cpp::execution_policy<Derived> {};
template <typename Derived>
struct device_execution_policy : thrust::system::hip::execution_policy<Derived> {};

typedef thrust::system::cpp::tag host_system_tag;
typedef thrust::system::hip::tag device_system_tag;

}  // namespace thrust
