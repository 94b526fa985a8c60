// thrust::host_memory_resource: where host_vector's storage comes from (thrust/mr/host_memory_resource.h:28-30).
#pragma once
#include <thrust/mr/new.h>

namespace thrust {
typedef thrust::mr::new_delete_resource host_memory_resource;
}  // namespace thrust
