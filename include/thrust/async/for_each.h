// thrust::async::for_each: f(x) for every element of a device range, enqueued on the policy's
// stream; returns a device_event (thrust/async/for_each.h:68-112 of the reference).  The
// functor runs in a kernel instantiated for it, so the calling translation unit is compiled
// with hipcc, as for the synchronous thrust::for_each with a user functor.
#pragma once
#include <thrust/future.h>
#include <thrust/transform.h>

namespace thrust {
namespace async {

template <typename D, typename It, typename F>
device_event for_each(const thrust::detail::execution_policy_base<D>& exec, It first, It last, F f) {
  namespace backend = thrust::system::hip::detail;
  static_assert(backend::is_device_output<It>::value,
                "thrust::async::for_each needs device_ptr / device_vector iterators, raw device pointers or a zip of them");
  auto& pol = thrust::detail::derived_cast(thrust::detail::strip_const(exec));
  backend::async_context ctx = backend::context_of(pol, 0);
  const uint64_t n = (uint64_t)(last - first);
#if defined(__HIPCC__)
  if (n != 0) {
    hipLaunchKernelGGL((backend::for_each_kernel<typename thrust::detail::device_view_of<It>::type, F>),
                       dim3(backend::elementwise_grid(n)), dim3(backend::ELEMENTWISE_BLOCK), 0, (hipStream_t)ctx.stream(),
                       thrust::detail::device_view(first), n, f);
    backend::throw_on_error(backend::launch_status(), "async::for_each: kernel launch");
  }
#else
  static_assert(backend::fancy_needs_hipcc<F>::value,
                "thrust::async::for_each runs the functor in a kernel; compile this translation unit with hipcc");
#endif
  return device_event(ctx.keep);
}
template <typename It, typename F,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<It>::value>::type>
device_event for_each(It first, It last, F f) {
  return thrust::async::for_each(thrust::device, first, last, f);
}

}  // namespace async
}  // namespace thrust
