// thrust_amd_merge / thrust_amd_merge_by_key: the library's instantiations of the merge-path
// merge (thrust/system/hip/detail/merge_kernels.h describes it).  Keys are compared by value
// with operator< (floats: IEEE, -0.0 == +0.0), descending = operator>.
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"
#include "../../include/thrust/system/hip/detail/merge_kernels.h"

namespace ta {
using namespace ::thrust::system::hip::merging;

// The direction is part of the type: a comparison is one instruction in the kernels' inner loops.
template <bool DESCENDING>
struct OrderComp {
  template <typename T>
  TA_DEVICE bool operator()(const T& x, const T& y) const { return DESCENDING ? (y < x) : (x < y); }
};

template <typename T, typename V, bool HAS_VALUES>
static int merge_run(void* temp, size_t* temp_bytes, const void* a, uint64_t na, const void* b,
                     uint64_t nb, const void* va, const void* vb, void* out, void* vout,
                     int descending, hipStream_t stream) {
  const uint64_t total = na + nb;
  const uint64_t tiles = (total + MERGE_TILE - 1) / MERGE_TILE;
  if (tiles > 0x7fffffffull) return (int)hipErrorInvalidValue;
  const size_t need = merge_temp_bytes(total);
  if (!temp) {
    *temp_bytes = need;
    return 0;
  }
  if (*temp_bytes < need) return (int)hipErrorInvalidValue;
  if (total == 0) return 0;
  if ((na && !a) || (nb && !b) || !out) return (int)hipErrorInvalidValue;
  if (HAS_VALUES && ((na && !va) || (nb && !vb) || !vout)) return (int)hipErrorInvalidValue;
  auto launch = [&](auto comp) {
    return merge_launch<T, V, HAS_VALUES>(static_cast<uint64_t*>(temp), static_cast<const T*>(a), na,
                                          static_cast<const T*>(b), nb, static_cast<const V*>(va),
                                          static_cast<const V*>(vb), static_cast<T*>(out), static_cast<V*>(vout),
                                          comp, stream);
  };
  return descending ? launch(OrderComp<true>{}) : launch(OrderComp<false>{});
}

}  // namespace ta

TA_EXPORT int thrust_amd_merge(void* temp, size_t* temp_bytes, const void* a, uint64_t na,
                               const void* b, uint64_t nb, void* out, int dtype, int descending,
                               void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(dtype)) return (int)hipErrorInvalidValue;
  return with_dtype(dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return merge_run<T, uint32_t, false>(temp, temp_bytes, a, na, b, nb, nullptr, nullptr, out, nullptr,
                                         descending, (hipStream_t)stream);
  });
}

TA_EXPORT int thrust_amd_merge_by_key(void* temp, size_t* temp_bytes, const void* keys_a, uint64_t na,
                                      const void* keys_b, uint64_t nb, const void* values_a,
                                      const void* values_b, void* keys_out, void* values_out,
                                      int key_dtype, size_t value_bytes, int descending, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype) || !valid_item_bytes(value_bytes))
    return (int)hipErrorInvalidValue;
  return with_dtype(key_dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_item_bytes(value_bytes, [&](auto vt) {
      using V = typename decltype(vt)::type;
      return merge_run<T, V, true>(temp, temp_bytes, keys_a, na, keys_b, nb, values_a, values_b,
                                   keys_out, values_out, descending, (hipStream_t)stream);
    });
  });
}
