// thrust_amd_reduce_by_key: the library's instantiations of the single-pass segmented
// reduction (thrust/system/hip/detail/reduce_by_key_kernels.h describes it) for keys compared
// with == and the operators of the C interface.
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"
#include "segmented.hpp"

namespace ta {

struct KeysEqual {
  template <typename K>
  TA_DEVICE bool operator()(const K& a, const K& b) const { return a == b; }
};

template <typename K, typename V, typename Op>
static int rbk_run(void* temp, size_t* temp_bytes, const void* keys_in, const void* values_in,
                   void* keys_out, void* values_out, uint64_t* d_num_runs, uint64_t n,
                   hipStream_t stream) {
  const RbkTemp<K, V> lay(n);
  if (lay.tiles > 0xffffffffull || n >= 0xffffffffull) return (int)hipErrorInvalidValue;
  if (!temp) {
    *temp_bytes = lay.total;
    return 0;
  }
  if (*temp_bytes < lay.total || !d_num_runs) return (int)hipErrorInvalidValue;
  if (n && (!keys_in || !values_in || !keys_out || !values_out)) return (int)hipErrorInvalidValue;
  RbkArgs<K, V, KeysEqual, Op> a = make_rbk_args<K, V>(KeysEqual{}, Op{});
  a.keys = static_cast<const K*>(keys_in);
  a.values = static_cast<const V*>(values_in);
  a.keys_out = static_cast<K*>(keys_out);
  a.values_out = static_cast<V*>(values_out);
  a.d_num_runs = d_num_runs;
  a.n = n;
  return rbk_launch(static_cast<char*>(temp), a, stream);
}

}  // namespace ta

TA_EXPORT int thrust_amd_reduce_by_key(void* temp, size_t* temp_bytes, const void* keys_in,
                                       const void* values_in, void* keys_out, void* values_out,
                                       uint64_t* d_num_runs, uint64_t n, int key_dtype,
                                       int value_dtype, int op, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype) || !valid_dtype(value_dtype) || !valid_binop(op))
    return (int)hipErrorInvalidValue;
  auto by_value = [&](auto kt) {
    using K = typename decltype(kt)::type;
    return with_dtype(value_dtype, [&](auto vt) {
      using V = typename decltype(vt)::type;
      return with_binop(op, [&](auto o) {
        return rbk_run<K, V, decltype(o)>(temp, temp_bytes, keys_in, values_in, keys_out, values_out,
                                          d_num_runs, n, (hipStream_t)stream);
      });
    });
  };
  if (key_dtype == THRUST_AMD_F32) return by_value(TypeTag<float>{});
  if (key_dtype == THRUST_AMD_F64) return by_value(TypeTag<double>{});
  return with_item_bytes(thrust_amd_dtype_size(key_dtype), by_value);
}
