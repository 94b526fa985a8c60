// thrust::device_event: see thrust/future.h.
#pragma once
#include <thrust/future.h>
