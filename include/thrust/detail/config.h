// Configuration of the MI355X-native Thrust front end.
//
// The device system is fixed: thrust::system::hip (alias thrust::hip), whose algorithms
// forward to the C ABI of libthrust_amd (include/thrust_amd.h).  The reference selects its
// device system with THRUST_DEVICE_SYSTEM (thrust/detail/config/device_system.h:20-60);
// here the macro is accepted and must name this system if it is defined at all.
#pragma once
#include <cassert>  // programs written for the reference get assert() from its headers

#define THRUST_DEVICE_SYSTEM_HIP 5
#ifndef THRUST_DEVICE_SYSTEM
#define THRUST_DEVICE_SYSTEM THRUST_DEVICE_SYSTEM_HIP
#endif
#if THRUST_DEVICE_SYSTEM != THRUST_DEVICE_SYSTEM_HIP
#error "this Thrust front end provides the HIP (gfx950) device system only"
#endif

// Same version number as the API surface it mirrors (thrust/version.h:50 of the reference).
#define THRUST_VERSION 101400
#define THRUST_MAJOR_VERSION (THRUST_VERSION / 100000)
#define THRUST_MINOR_VERSION (THRUST_VERSION / 100 % 1000)
#define THRUST_SUBMINOR_VERSION (THRUST_VERSION % 100)
#define THRUST_PATCH_NUMBER 0

// User code written for the reference decorates functors with these.
#ifndef __host__
#define __host__
#endif
#ifndef __device__
#define __device__
#endif

// Written between a function's name and its parameter list where <windows.h>-style min / max
// macros would otherwise expand: `min THRUST_AMD_NO_MACRO (a, b)`.
#ifndef THRUST_AMD_NO_MACRO
#define THRUST_AMD_NO_MACRO
#endif
// the reference's name for the same thing (thrust/detail/config/config.h)
#ifndef THRUST_PREVENT_MACRO_SUBSTITUTION
#define THRUST_PREVENT_MACRO_SUBSTITUTION
#endif
