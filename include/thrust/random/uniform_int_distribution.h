// thrust::random::uniform_int_distribution under the reference's header name (thrust/random/uniform_int_distribution.h).
#pragma once
#include <thrust/random.h>
