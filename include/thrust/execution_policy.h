// thrust::host, thrust::device, thrust::seq, thrust::hip::par, par.on(stream).
#pragma once
#include <thrust/detail/execution_policy.h>

namespace thrust {
namespace detail {
struct host_t : thrust::host_execution_policy<host_t> {};
struct device_t : thrust::device_execution_policy<device_t> {};
struct seq_t : thrust::system::cpp::execution_policy<seq_t> {};
}  // namespace detail

static const detail::host_t host;
static const detail::device_t device;
static const detail::seq_t seq;

namespace system {
namespace hip {

// Policy bound to a stream: thrust::hip::par.on(stream).
struct stream_policy : execution_policy<stream_policy> {
  void* stream;
  explicit stream_policy(void* s) : stream(s) {}
};
inline void* get_stream(const stream_policy& p) { return p.stream; }

struct par_t : execution_policy<par_t> {
  // `stream` is a hipStream_t; it is taken as void* so that user code needs no HIP headers.
  stream_policy on(void* stream) const { return stream_policy(stream); }
};
static const par_t par;

namespace detail {
// The stream of any policy of this system: the most derived get_stream wins.
template <typename Derived>
inline void* stream_of(execution_policy<Derived>& p) {
  return get_stream(thrust::detail::derived_cast(p));
}
}  // namespace detail

}  // namespace hip
}  // namespace system

namespace hip = system::hip;
namespace cpp {
using thrust::system::cpp::execution_policy;
using thrust::system::cpp::tag;
static const thrust::detail::seq_t par;
}  // namespace cpp

}  // namespace thrust
