// thrust::async::transform: output[i] = f(input[i]) over a device range, enqueued on the
// policy's stream; returns a device_event (thrust/async/transform.h:70-118 of the reference).
// The functor runs in a kernel instantiated for it (hipcc translation units).
#pragma once
#include <thrust/future.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/transform.h>

namespace thrust {
namespace async {

template <typename D, typename In, typename Out, typename F>
device_event transform(const thrust::detail::execution_policy_base<D>& exec, In first, In last, Out output, F f) {
  namespace backend = thrust::system::hip::detail;
  static_assert(backend::is_device_input<In>::value && backend::is_device_output<Out>::value,
                "thrust::async::transform reads device or fancy iterators and writes device memory");
  auto& pol = thrust::detail::derived_cast(thrust::detail::strip_const(exec));
  backend::async_context ctx = backend::context_of(pol, 0);
  const uint64_t n = (uint64_t)(last - first);
  // the kernel that writes a fancy iterator out evaluates f once per element, straight into the output
  backend::materialize(ctx.stream(), thrust::make_transform_iterator(first, f), output, n);
  return device_event(ctx.keep);
}
template <typename In, typename Out, typename F,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<In>::value>::type>
device_event transform(In first, In last, Out output, F f) {
  return thrust::async::transform(thrust::device, first, last, output, f);
}

}  // namespace async
}  // namespace thrust
