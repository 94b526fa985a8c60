// thrust_amd_inclusive_scan / thrust_amd_exclusive_scan: the single-pass scan kernel of
// scan_kernel.hpp on the untransformed input.  Replaces cub::DispatchScan as called from
// thrust/system/cuda/detail/scan.h:55-200.
#include "scan_kernel.hpp"

#include <atomic>

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
namespace ta {

constexpr size_t SCAN_STATIC_SCRATCH_BYTES = (size_t)1 << 20;
static __device__ __align__(256) unsigned char scan_static_scratch[SCAN_STATIC_SCRATCH_BYTES];

constexpr int SCAN_STATIC_MAX_DEVICES = 64;
static std::atomic<void*> g_scan_scratch_ptr[SCAN_STATIC_MAX_DEVICES];

// Device address of the scratch array on the current device; every device holds its own copy.
static int scan_static_scratch_ptr(void** out) {
  int device = 0;
  TA_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= SCAN_STATIC_MAX_DEVICES) return (int)hipErrorInvalidDevice;
  void* p = g_scan_scratch_ptr[device].load(std::memory_order_acquire);
  if (!p) {
    TA_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scan_static_scratch)));
    if (!p) return (int)hipErrorInvalidSymbol;
    // two threads may both ask; they receive the same address
    g_scan_scratch_ptr[device].store(p, std::memory_order_release);
  }
  *out = p;
  return 0;
}

}  // namespace ta

TA_EXPORT int thrust_amd_inclusive_scan_static(const void* in, void* out, uint64_t n, int dtype,
                                               int op, void* stream) {
  using namespace ta;
  size_t need = 0;
  const int rc = thrust_amd_inclusive_scan(nullptr, &need, in, out, n, dtype, op, stream);
  if (rc) return rc;
  if (need > SCAN_STATIC_SCRATCH_BYTES) return (int)hipErrorInvalidValue;  // n beyond the fixed scratch
  void* scratch = nullptr;
  const int rs = scan_static_scratch_ptr(&scratch);
  if (rs) return rs;
  size_t bytes = SCAN_STATIC_SCRATCH_BYTES;
  return thrust_amd_inclusive_scan(scratch, &bytes, in, out, n, dtype, op, stream);
}
