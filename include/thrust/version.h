#pragma once
#include <thrust/detail/config.h>
