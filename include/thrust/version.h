// The version of the API surface this front end mirrors (thrust/version.h:50-75).
#pragma once
#include <thrust/detail/config.h>
