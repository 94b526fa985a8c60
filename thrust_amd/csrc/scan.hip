// thrust_amd_inclusive_scan / thrust_amd_exclusive_scan: the single-pass scan kernel of
// scan_kernel.hpp on the untransformed input.  Replaces cub::DispatchScan as called from
// thrust/system/cuda/detail/scan.h:55-200.
#include "scan_kernel.hpp"

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
