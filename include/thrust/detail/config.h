// Configuration of the MI355X-native Thrust front end.
//
// The device system is fixed: thrust::system::hip (alias thrust::hip), whose algorithms
// forward to the C ABI of libthrust_amd (include/thrust_amd.h).  The reference selects its
// device system with THRUST_DEVICE_SYSTEM (thrust/detail/config/device_system.h:20-60);
// here the macro is accepted and must name this system if it is defined at all.
#pragma once

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

// User code written for the reference decorates functors with these.
#ifndef __host__
#define __host__
#endif
#ifndef __device__
#define __device__
#endif
