// thrust::random::discard_block_engine under the reference's header name (thrust/random/discard_block_engine.h).
#pragma once
#include <thrust/random.h>
