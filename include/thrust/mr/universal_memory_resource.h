// thrust::universal_memory_resource under the reference's header name (thrust/mr/universal_memory_resource.h).
#pragma once
#include <thrust/universal_vector.h>
