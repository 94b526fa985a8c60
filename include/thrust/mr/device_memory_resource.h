// thrust::device_memory_resource under the reference's header name (thrust/mr/device_memory_resource.h).
#pragma once
#include <thrust/device_allocator.h>
