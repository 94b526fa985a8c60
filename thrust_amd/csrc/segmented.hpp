// Pieces shared by the segmented single-pass kernels (reduce_by_key, scan_by_key): the
// (heads, value) pair, its associative operator, the value vector that travels with a
// 16-byte vector of keys, and the tile shapes.  They live in the header that also holds the
// reduce_by_key kernel template, which users' translation units instantiate as well.
#pragma once
#include "common.hpp"
#include "launch.hpp"
#include "../../include/thrust/system/hip/detail/reduce_by_key_kernels.h"

namespace ta {
using namespace ::thrust::system::hip::segmented;

}  // namespace ta
