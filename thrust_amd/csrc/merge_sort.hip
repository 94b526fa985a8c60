// thrust_amd_merge_sort_keys / thrust_amd_merge_sort_pairs: the stable comparison sort
// instantiated for the two orders a C ABI can name, operator< and operator> on the ten
// arithmetic key types.  The kernels and the pass driver are the header templates that
// user translation units instantiate for their own comparators; here every launch also
// goes through the library's per-kernel timers.
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"

#define THRUST_AMD_MERGE_SORT_LAUNCH(label, stream, kernel, grid, block, ...) \
  TA_LAUNCH(label, stream, kernel, grid, block, __VA_ARGS__)
#include "../../include/thrust/system/hip/detail/merge_sort_kernels.h"

namespace ta {

struct CompLess {
  template <typename T>
  TA_DEVICE bool operator()(const T& a, const T& b) const { return a < b; }
};
struct CompGreater {
  template <typename T>
  TA_DEVICE bool operator()(const T& a, const T& b) const { return b < a; }
};

template <typename K, typename V, bool HAS_VALUES>
static int merge_sort_run(void* temp, size_t* temp_bytes, void* keys, void* values, uint64_t n, int descending,
                          hipStream_t stream) {
  namespace ms = thrust::system::hip::merge_sort;
  if (descending)
    return ms::sort<K, V, HAS_VALUES>(temp, temp_bytes, static_cast<K*>(keys), static_cast<V*>(values), n,
                                      CompGreater{}, stream);
  return ms::sort<K, V, HAS_VALUES>(temp, temp_bytes, static_cast<K*>(keys), static_cast<V*>(values), n, CompLess{},
                                    stream);
}

}  // namespace ta

TA_EXPORT int thrust_amd_merge_sort_keys(void* temp, size_t* temp_bytes, void* keys, uint64_t n, int key_dtype,
                                         int descending, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype)) return (int)hipErrorInvalidValue;
  return with_dtype(key_dtype, [&](auto tt) {
    using K = typename decltype(tt)::type;
    return merge_sort_run<K, uint32_t, false>(temp, temp_bytes, keys, nullptr, n, descending, (hipStream_t)stream);
  });
}

TA_EXPORT int thrust_amd_merge_sort_pairs(void* temp, size_t* temp_bytes, void* keys, void* values, uint64_t n,
                                          int key_dtype, size_t value_bytes, int descending, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype) || !valid_item_bytes(value_bytes)) return (int)hipErrorInvalidValue;
  return with_dtype(key_dtype, [&](auto tt) {
    using K = typename decltype(tt)::type;
    return with_item_bytes(value_bytes, [&](auto vt) {
      using V = typename decltype(vt)::type;
      return merge_sort_run<K, V, true>(temp, temp_bytes, keys, values, n, descending, (hipStream_t)stream);
    });
  });
}
