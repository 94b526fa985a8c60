// thrust::random::normal_distribution under the reference's header name (thrust/random/normal_distribution.h).
#pragma once
#include <thrust/random.h>
