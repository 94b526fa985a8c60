// thrust::mr::tls_pool: one unsynchronized pool per thread over an upstream resource
// (thrust/mr/tls_pool.h:40-58).  The upstream named on a thread's first call is the one its pool keeps.
#pragma once
#include <thrust/mr/memory_resource.h>
#include <thrust/mr/pool.h>

namespace thrust {
namespace mr {
template <typename Upstream>
inline unsynchronized_pool_resource<Upstream>& tls_pool(Upstream* upstream = nullptr) {
  static thread_local unsynchronized_pool_resource<Upstream> pool(upstream ? upstream : get_global_resource<Upstream>());
  return pool;
}
}  // namespace mr
}  // namespace thrust
