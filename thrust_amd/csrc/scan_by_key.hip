// thrust_amd_inclusive_scan_by_key / thrust_amd_exclusive_scan_by_key: the library's
// instantiations of the single-pass segmented scan
// (thrust/system/hip/detail/scan_by_key_kernels.h describes it) for keys compared with == and
// the operators of the C interface.
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"
#include "segmented.hpp"
#include "../../include/thrust/system/hip/detail/scan_by_key_kernels.h"

namespace ta {

struct SbkKeysEqual {
  template <typename K>
  TA_DEVICE bool operator()(const K& a, const K& b) const { return a == b; }
};

template <typename K, typename V, typename Op>
static int sbk_run(void* temp, size_t* temp_bytes, const void* keys, const void* values, void* out,
                   uint64_t n, bool exclusive, const void* init, hipStream_t stream) {
  const SbkTemp<K, V> lay(n);
  if (lay.tiles > 0xffffffffull || n >= 0xffffffffull) return (int)hipErrorInvalidValue;
  if (!temp) {
    *temp_bytes = lay.total;
    return 0;
  }
  if (*temp_bytes < lay.total || (exclusive && !init)) return (int)hipErrorInvalidValue;
  if (n == 0) return 0;
  if (!keys || !values || !out) return (int)hipErrorInvalidValue;
  V init_v{};
  if (exclusive) __builtin_memcpy(&init_v, init, sizeof(V));
  return sbk_launch(static_cast<char*>(temp), static_cast<const K*>(keys), static_cast<const V*>(values),
                    static_cast<V*>(out), n, exclusive, init_v, SbkKeysEqual{}, Op{}, stream);
}

static int sbk_dispatch(void* temp, size_t* temp_bytes, const void* keys, const void* values, void* out,
                        uint64_t n, int key_dtype, int value_dtype, int op, bool exclusive,
                        const void* init, hipStream_t stream) {
  if (!temp_bytes || !valid_dtype(key_dtype) || !valid_dtype(value_dtype) || !valid_binop(op))
    return (int)hipErrorInvalidValue;
  auto by_value = [&](auto kt) {
    using K = typename decltype(kt)::type;
    return with_dtype(value_dtype, [&](auto vt) {
      using V = typename decltype(vt)::type;
      return with_binop(op, [&](auto o) {
        return sbk_run<K, V, decltype(o)>(temp, temp_bytes, keys, values, out, n, exclusive, init, stream);
      });
    });
  };
  if (key_dtype == THRUST_AMD_F32) return by_value(TypeTag<float>{});
  if (key_dtype == THRUST_AMD_F64) return by_value(TypeTag<double>{});
  return with_item_bytes(thrust_amd_dtype_size(key_dtype), by_value);
}

}  // namespace ta

TA_EXPORT int thrust_amd_inclusive_scan_by_key(void* temp, size_t* temp_bytes, const void* keys,
                                               const void* values, void* out, uint64_t n, int key_dtype,
                                               int value_dtype, int op, void* stream) {
  return ta::sbk_dispatch(temp, temp_bytes, keys, values, out, n, key_dtype, value_dtype, op, false, nullptr,
                          (hipStream_t)stream);
}

TA_EXPORT int thrust_amd_exclusive_scan_by_key(void* temp, size_t* temp_bytes, const void* keys,
                                               const void* values, void* out, uint64_t n, int key_dtype,
                                               int value_dtype, int op, const void* init, void* stream) {
  return ta::sbk_dispatch(temp, temp_bytes, keys, values, out, n, key_dtype, value_dtype, op, true, init,
                          (hipStream_t)stream);
}
