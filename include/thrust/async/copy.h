// thrust::async::copy.
//
// copy(policy, first, last, output) between device ranges is enqueued on the policy's stream
// and returns a device_event (thrust/async/copy.h of the reference).  A copy to or from host
// memory is made with the blocking transfer of thrust::copy -- pageable host memory is
// staged by the runtime in any case -- after the policy's dependencies have finished, and
// the event returned is complete.
#pragma once
#include <thrust/copy.h>
#include <thrust/future.h>

namespace thrust {
namespace async {

template <typename D, typename In, typename Out>
device_event copy(const thrust::detail::execution_policy_base<D>& exec, In first, In last, Out output) {
  namespace backend = thrust::system::hip::detail;
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  auto& pol = thrust::detail::derived_cast(thrust::detail::strip_const(exec));
  backend::async_context ctx = backend::context_of(pol, 0);
  const bool in_device = std::is_pointer<In>::value ? true : thrust::detail::is_device_iterator<In>::value;
  const bool out_device = std::is_pointer<Out>::value ? true : thrust::detail::is_device_iterator<Out>::value;
  (void)sizeof(T);
  thrust::detail::copy_dispatch(first, last, output, in_device, out_device, ctx.stream(), false);
  return device_event(ctx.keep);
}
template <typename In, typename Out,
          typename = typename std::enable_if<!thrust::detail::is_execution_policy<In>::value>::type>
device_event copy(In first, In last, Out output) {
  return thrust::async::copy(thrust::device, first, last, output);
}

}  // namespace async
}  // namespace thrust
