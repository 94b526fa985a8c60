// thrust/universal_allocator.h of the reference: here the allocator lives in thrust/universal_vector.h.
#pragma once
#include <thrust/universal_vector.h>
