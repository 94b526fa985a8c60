// Kernel launch wrapper.  TA_LAUNCH(label, stream, kernel, grid, block, args...) enqueues
// the kernel; when per-kernel timing has been switched on (thrust_amd_profile_enable) it
// also brackets the launch with two events on the same stream.  Timing is a debugging
// aid in the spirit of the reference's THRUST_DEBUG_SYNC per-launch log
// (thrust/system/cuda/detail/core/agent_launcher.h:518-535); it is off by default and
// costs one relaxed load per launch when off.
#pragma once
#include "common.hpp"

namespace ta {

bool profile_on();
void profile_mark(const char* label, hipStream_t stream, bool begin);

struct LaunchTimer {
  const char* label;
  hipStream_t stream;
  bool on;
  LaunchTimer(const char* l, hipStream_t s) : label(l), stream(s), on(profile_on()) {
    if (on) profile_mark(label, stream, true);
  }
  ~LaunchTimer() {
    if (on) profile_mark(label, stream, false);
  }
};

}  // namespace ta

#define TA_LAUNCH(label, stream, kernel, grid, block, ...)                         \
  do {                                                                             \
    ta::LaunchTimer _ta_timer(label, stream);                                      \
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__);               \
  } while (0)
