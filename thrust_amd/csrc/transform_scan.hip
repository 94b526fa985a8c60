// thrust_amd_transform_inclusive_scan / thrust_amd_transform_exclusive_scan: the single-pass
// scan kernel of scan_kernel.hpp with negate or square applied to every element as it is
// loaded (the identity is routed to the plain scans).  The reference scans a transform
// iterator the same way (thrust/system/cuda/detail/transform_scan.h:39-115): the input is
// read once, nothing is staged.
// (The inclusive and the exclusive form sit in two files so that they compile side by side.)
#include "scan_kernel.hpp"

namespace ta {

template <bool EXCLUSIVE>
static int transform_scan(void* temp, size_t* temp_bytes, const void* in, void* out, uint64_t n,
                          int dtype, int unary, int op, const void* init, hipStream_t stream) {
  return with_transform(unary, [&](auto un) {
    using Un = decltype(un);
    return dispatch_dtype_op<ScanLaunch<EXCLUSIVE, Un>>(dtype, op, temp, temp_bytes, in, out, n, init,
                                                        stream);
  });
}

}  // namespace ta

TA_EXPORT int thrust_amd_transform_inclusive_scan(void* temp, size_t* temp_bytes, const void* in,
                                                  void* out, uint64_t n, int dtype, int unary,
                                                  int op, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(dtype) || !valid_unary(unary) || !valid_binop(op))
    return (int)hipErrorInvalidValue;
  if (unary == THRUST_AMD_IDENTITY)
    return thrust_amd_inclusive_scan(temp, temp_bytes, in, out, n, dtype, op, stream);
  return transform_scan<false>(temp, temp_bytes, in, out, n, dtype, unary, op, nullptr,
                               (hipStream_t)stream);
}
