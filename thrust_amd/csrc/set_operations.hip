// thrust_amd_set_operation / thrust_amd_set_operation_by_key: the library's instantiations of
// the single-pass set operations (thrust/system/hip/detail/set_operation_kernels.h describes
// them).  Keys are compared with operator< (descending: operator>).
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"
#include "../../include/thrust/system/hip/detail/set_operation_kernels.h"

namespace ta {
using namespace ::thrust::system::hip::setops;

// The direction is part of the type: a comparison is one instruction in the kernels' inner loops.
template <bool DESCENDING>
struct SetOrder {
  template <typename T>
  TA_DEVICE bool operator()(const T& x, const T& y) const { return DESCENDING ? (y < x) : (x < y); }
};

template <typename T, typename V, bool HAS_VALUES>
static int set_run(void* temp, size_t* temp_bytes, int op, const void* a, uint64_t na, const void* b,
                   uint64_t nb, const void* va, const void* vb, void* out, void* vout,
                   uint64_t* d_num, int descending, hipStream_t stream) {
  const uint64_t total = na + nb;
  const SetTemp<T, V, HAS_VALUES> lay(total);
  if (lay.tiles > 0x7fffffffull) return (int)hipErrorInvalidValue;
  if (!temp) {
    *temp_bytes = lay.total;
    return 0;
  }
  if (*temp_bytes < lay.total || !d_num) return (int)hipErrorInvalidValue;
  if ((na && !a) || (nb && !b) || (total && !out)) return (int)hipErrorInvalidValue;
  // values of B are read only by the two operations that can keep an element of B
  const bool keeps_b = op == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE || op == THRUST_AMD_SET_UNION;
  if (HAS_VALUES && ((na && !va) || (nb && keeps_b && !vb) || (total && !vout)))
    return (int)hipErrorInvalidValue;
  auto launch = [&](auto comp) {
    return set_launch<T, V, HAS_VALUES>(static_cast<char*>(temp), op, static_cast<const T*>(a), na,
                                        static_cast<const T*>(b), nb, static_cast<const V*>(va),
                                        static_cast<const V*>(vb), static_cast<T*>(out), static_cast<V*>(vout), d_num,
                                        comp, stream);
  };
  return descending ? launch(SetOrder<true>{}) : launch(SetOrder<false>{});
}

inline bool valid_set_op(int op) { return op >= 0 && op < THRUST_AMD_SET_OP_COUNT; }

}  // namespace ta

TA_EXPORT int thrust_amd_set_operation(void* temp, size_t* temp_bytes, int op, const void* a, uint64_t na,
                                       const void* b, uint64_t nb, void* out, uint64_t* d_num_out,
                                       int dtype, int descending, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(dtype) || !valid_set_op(op)) return (int)hipErrorInvalidValue;
  return with_dtype(dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return set_run<T, uint32_t, false>(temp, temp_bytes, op, a, na, b, nb, nullptr, nullptr, out, nullptr,
                                       d_num_out, descending, (hipStream_t)stream);
  });
}

TA_EXPORT int thrust_amd_set_operation_by_key(void* temp, size_t* temp_bytes, int op, const void* keys_a,
                                              uint64_t na, const void* keys_b, uint64_t nb,
                                              const void* values_a, const void* values_b, void* keys_out,
                                              void* values_out, uint64_t* d_num_out, int key_dtype,
                                              size_t value_bytes, int descending, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype) || !valid_item_bytes(value_bytes) || !valid_set_op(op))
    return (int)hipErrorInvalidValue;
  return with_dtype(key_dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_item_bytes(value_bytes, [&](auto vt) {
      using V = typename decltype(vt)::type;
      return set_run<T, V, true>(temp, temp_bytes, op, keys_a, na, keys_b, nb, values_a, values_b, keys_out,
                                 values_out, d_num_out, descending, (hipStream_t)stream);
    });
  });
}
