// thrust::random::linear_congruential_engine under the reference's header name (thrust/random/linear_congruential_engine.h).
#pragma once
#include <thrust/random.h>
