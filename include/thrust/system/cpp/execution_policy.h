// thrust::cpp::par, thrust::cpp::tag: the sequential host system (thrust/system/cpp/execution_policy.h).
#pragma once
#include <thrust/execution_policy.h>
