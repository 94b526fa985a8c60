// thrust/device_malloc.h of the reference: here the declarations live in thrust/device_ptr.h.
#pragma once
#include <thrust/device_ptr.h>
