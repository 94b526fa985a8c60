// thrust::random::xor_combine_engine under the reference's header name (thrust/random/xor_combine_engine.h).
#pragma once
#include <thrust/random.h>
