// thrust::mr::pool_options under the reference's header name (thrust/mr/pool_options.h).
#pragma once
#include <thrust/mr/pool.h>
