// thrust::random::uniform_real_distribution under the reference's header name (thrust/random/uniform_real_distribution.h).
#pragma once
#include <thrust/random.h>
