// thrust::system::system_error under the reference's header name (thrust/system/system_error.h).
#pragma once
#include <thrust/system_error.h>
