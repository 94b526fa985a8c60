// thrust::random::subtract_with_carry_engine under the reference's header name (thrust/random/subtract_with_carry_engine.h).
#pragma once
#include <thrust/random.h>
