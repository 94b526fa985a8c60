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
// Records an event on the stream and returns it (null on failure).
hipEvent_t profile_begin(hipStream_t stream);
// Records the closing event and files the pair under the label.
void profile_end(const char* label, hipStream_t stream, hipEvent_t begin);

// The opening event lives in the timer object, so launches from several host threads do
// not mix their brackets.
struct LaunchTimer {
  const char* label;
  hipStream_t stream;
  hipEvent_t begin;
  LaunchTimer(const char* l, hipStream_t s) : label(l), stream(s), begin(profile_on() ? profile_begin(s) : nullptr) {}
  ~LaunchTimer() {
    if (begin) profile_end(label, stream, begin);
  }
};

}  // namespace ta

#define TA_LAUNCH(label, stream, kernel, grid, block, ...)                         \
  do {                                                                             \
    ta::LaunchTimer _ta_timer(label, stream);                                      \
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__);               \
  } while (0)
