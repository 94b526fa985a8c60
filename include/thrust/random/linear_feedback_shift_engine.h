// thrust::random::linear_feedback_shift_engine under the reference's header name (thrust/random/linear_feedback_shift_engine.h).
#pragma once
#include <thrust/random.h>
