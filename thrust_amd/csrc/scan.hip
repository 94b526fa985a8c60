// thrust_amd_inclusive_scan / thrust_amd_exclusive_scan: the single-pass scan kernel of
// scan_kernel.hpp on the untransformed input.  Replaces cub::DispatchScan as called from
// thrust/system/cuda/detail/scan.h:55-200.
#include "scan_kernel.hpp"

#include <mutex>

TA_EXPORT int thrust_amd_inclusive_scan(void* temp, size_t* temp_bytes, const void* in, void* out,
                                         uint64_t n, int dtype, int op, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(dtype) || !valid_binop(op)) return (int)hipErrorInvalidValue;
  return dispatch_dtype_op<ScanLaunch<false, UnIdentity>>(dtype, op, temp, temp_bytes, in, out, n,
                                                          (const void*)nullptr, (hipStream_t)stream);
}

TA_EXPORT int thrust_amd_exclusive_scan(void* temp, size_t* temp_bytes, const void* in, void* out,
                                         uint64_t n, int dtype, int op, const void* init,
                                         void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(dtype) || !valid_binop(op)) return (int)hipErrorInvalidValue;
  return dispatch_dtype_op<ScanLaunch<true, UnIdentity>>(dtype, op, temp, temp_bytes, in, out, n,
                                                         init, (hipStream_t)stream);
}

// ------------------------------------------------------------------ scan without allocation
// thrust_amd_inclusive_scan_static: the inclusive scan for callers that cannot allocate.
// The tile descriptors and the ticket live in a fixed array inside the library's own device
// image instead of caller-provided temporary storage.  In host code the array's name is a
// host-side stand-in, not a device address: its address on the current device is asked for
// once per device (hipGetSymbolAddress) and that pointer is what the kernels receive.
//
// The array is all zero when the module is loaded and every scan leaves it all zero again (the
// tile that finishes last clears what the call used), so no clearing kernel runs in front of the
// scan.  Calls on one GPU share the array: a per-device event, recorded behind every call and waited
// for by the next call's stream, keeps them one after the other on the device, and a mutex keeps
// the host side of two threads apart.  A stream that is being captured takes no part in that
// (events of other work cannot enter a capture): replays of such a graph must not overlap other
// calls of this entry point on the same GPU.
namespace ta {

constexpr size_t SCAN_STATIC_SCRATCH_BYTES = (size_t)1 << 20;
static __device__ __align__(256) unsigned char scan_static_scratch[SCAN_STATIC_SCRATCH_BYTES];

constexpr int SCAN_STATIC_MAX_DEVICES = 64;
struct ScanStaticDevice {
  std::mutex lock;
  void* scratch = nullptr;    // device address of the array on this device
  hipEvent_t last = nullptr;  // recorded behind the latest call
  hipStream_t last_stream = nullptr;  // ... on this stream (compared, never used)
  bool recorded = false;
  bool dirty = false;         // a launch failed: the array is cleared whole before the next use
};
static ScanStaticDevice g_scan_static[SCAN_STATIC_MAX_DEVICES];

// Set-up, once per device with that device current: the array's device address and the event.
static int scan_static_setup(ScanStaticDevice& dev) {
  if (dev.scratch) return 0;
  void* p = nullptr;
  TA_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scan_static_scratch)));
  if (!p) return (int)hipErrorInvalidSymbol;
  TA_CHECK(hipEventCreateWithFlags(&dev.last, hipEventDisableTiming));
  dev.scratch = p;
  return 0;
}

struct ScanStaticLaunch {
  template <typename T, typename Op>
  static int run(void* scratch, const void* in, void* out, uint64_t n, hipStream_t stream) {
    size_t bytes = SCAN_STATIC_SCRATCH_BYTES;
    return ScanLaunch<false, UnIdentity>::run<T, Op>(scratch, &bytes, in, out, n, nullptr, stream,
                                                     /*kept_clean=*/true);
  }
};

}  // namespace ta

TA_EXPORT int thrust_amd_inclusive_scan_static(const void* in, void* out, uint64_t n, int dtype,
                                               int op, void* stream) {
  using namespace ta;
  size_t need = 0;
  const int rc = thrust_amd_inclusive_scan(nullptr, &need, in, out, n, dtype, op, stream);
  if (rc) return rc;
  if (need > SCAN_STATIC_SCRATCH_BYTES) return (int)hipErrorInvalidValue;  // n beyond the fixed scratch
  if (n == 0) return 0;
  if (!in || !out) return (int)hipErrorInvalidValue;
  int device = 0;
  TA_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= SCAN_STATIC_MAX_DEVICES) return (int)hipErrorInvalidDevice;
  ScanStaticDevice& dev = g_scan_static[device];
  std::lock_guard<std::mutex> guard(dev.lock);
  if (!dev.scratch) {
    // The set-up calls are not stream work.  Should this first call come from a thread that is
    // capturing a stream, they run under the relaxed capture mode, which allows them there.
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    const bool exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    const int rs = scan_static_setup(dev);
    if (exchanged) (void)hipThreadExchangeStreamCaptureMode(&mode);
    if (rs) return rs;
  }
  hipStream_t s = (hipStream_t)stream;
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &capture) != hipSuccess) capture = hipStreamCaptureStatusNone;
  const bool ordered = capture == hipStreamCaptureStatusNone;
  // (a call on the stream of the call before it follows it anyway)
  if (ordered && dev.recorded && dev.last_stream != s) TA_CHECK(hipStreamWaitEvent(s, dev.last, 0));
  if (dev.dirty) {
    const uint64_t words = SCAN_STATIC_SCRATCH_BYTES / sizeof(uint64_t);
    TA_LAUNCH("tile_state_init", s, tile_state_init_kernel, dim3((uint32_t)((words + 255) / 256)), dim3(256),
              static_cast<uint64_t*>(dev.scratch), words, static_cast<uint32_t*>(dev.scratch), 0u);
    TA_CHECK_LAUNCH();
    dev.dirty = false;
  }
  const int status = dispatch_dtype_op<ScanStaticLaunch>(dtype, op, dev.scratch, in, out, n, s);
  if (status) {
    dev.dirty = true;
    return status;
  }
  if (ordered) {
    TA_CHECK(hipEventRecord(dev.last, s));
    dev.last_stream = s;
    dev.recorded = true;
  }
  return 0;
}
