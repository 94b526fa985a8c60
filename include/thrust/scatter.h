// thrust::scatter lives with the other element-wise algorithms.
#pragma once
#include <thrust/transform.h>
