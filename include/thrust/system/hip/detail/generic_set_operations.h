// set_difference, set_intersection, set_symmetric_difference, set_union and their _by_key
// forms for a user's comparator or key struct (hipcc translation units): the library's
// single-pass kernels over the merge path (thrust/system/hip/detail/set_operation_kernels.h),
// instantiated here for the comparator and the key type, as the reference passes the comparator
// into its agent (thrust/system/cuda/detail/set_operations.h:1480-1960).  Keys and values are
// items of 1, 2, 4 or 8 bytes.
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/hip/detail/generic_set_operations.h is HIP code: compile this translation unit with hipcc"
#endif
#include <thrust/pair.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/system/hip/detail/generic_by_key.h>
#include <thrust/system/hip/detail/set_operation_kernels.h>

namespace thrust {
namespace system {
namespace hip {
namespace detail {

// A range as an array of V: where it lies if it is one already, else a copy (converted) in `holder`.
template <typename V, typename It>
const V* values_as(void* stream, const temp_source& source, It first, uint64_t n, device_input<It>& direct,
                   temp_storage& holder, std::true_type) {
  (void)stream; (void)source; (void)first; (void)n; (void)holder;
  return (const V*)direct.ptr();
}
template <typename V, typename It>
const V* values_as(void* stream, const temp_source&, It first, uint64_t n, device_input<It>&, temp_storage& holder,
                   std::false_type) {
  if (n == 0) return nullptr;
  holder.ensure((std::size_t)n * sizeof(V));
  materialize(stream, first, static_cast<V*>(holder.ptr()), n);
  return static_cast<const V*>(holder.ptr());
}

// vf2 is not read when the operation never keeps an element of the second range.
template <int OP, typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,
          typename Comp>
uint64_t set_operation_generic(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko,
                               VOut vo, Comp comp, bool has_values) {
  namespace so = ::thrust::system::hip::setops;
  typedef typename std::remove_const<typename iterator_value<K1>::type>::type K;
  typedef typename iterator_value<VOut>::type V;
  typedef typename std::remove_const<typename iterator_value<V1>::type>::type Va;
  typedef typename std::remove_const<typename iterator_value<V2>::type>::type Vb;
  static_assert(is_abi_item<K>::value && std::is_same<typename iterator_value<KOut>::type, K>::value &&
                    std::is_same<typename std::remove_const<typename iterator_value<K2>::type>::type, K>::value,
                "set operations on the device system: keys of 1, 2, 4 or 8 bytes, one type for both inputs and the output");
  static_assert(is_abi_item<V>::value, "set operations by key on the device system: values of 1, 2, 4 or 8 bytes");
  void* stream = stream_of(exec);
  const temp_source source = temp_source_of(exec);
  const uint64_t na = (uint64_t)(kl1 - kf1), nb = (uint64_t)(kl2 - kf2), n = na + nb;
  if (n == 0) return 0;
  const bool keeps_second = OP == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE || OP == THRUST_AMD_SET_UNION;
  device_input<K1> a(stream, source, kf1, na);
  device_input<K2> b(stream, source, kf2, nb);
  temp_storage temp(stream, source);
  int rc;
  uint64_t* d_num;
  if (has_values) {
    const uint64_t nvb = keeps_second ? nb : 0;
    // inputs of the output's value type are read where they lie (fancy iterators are written
    // out first); inputs of another type are converted into temporary storage
    device_input<V1> da(stream, source, vf1, std::is_same<Va, V>::value ? na : 0);
    device_input<V2> db(stream, source, vf2, std::is_same<Vb, V>::value ? nvb : 0);
    temp_storage ha(stream, source), hb(stream, source);
    const V* va = values_as<V>(stream, source, vf1, na, da, ha, std::is_same<Va, V>());
    const V* vb = values_as<V>(stream, source, vf2, nvb, db, hb, std::is_same<Vb, V>());
    const so::SetTemp<K, V, true> lay(n);
    temp.ensure(lay.total + 256);
    char* base = static_cast<char*>(temp.ptr());
    d_num = reinterpret_cast<uint64_t*>(base + lay.total);
    rc = so::set_launch<K, V, true>(base, (int)OP, (const K*)a.ptr(), na, (const K*)b.ptr(), nb, va, vb,
                                    thrust::detail::raw(ko), (V*)thrust::detail::raw(vo), d_num, comp, (hipStream_t)stream);
    throw_on_error(rc, "set operation by key failed");
    return read_scalar<uint64_t>(d_num, stream, "set operation by key failed");  // blocks: the holders are idle after it
  }
  const so::SetTemp<K, uint32_t, false> lay(n);
  temp.ensure(lay.total + 256);
  char* base = static_cast<char*>(temp.ptr());
  d_num = reinterpret_cast<uint64_t*>(base + lay.total);
  rc = so::set_launch<K, uint32_t, false>(base, (int)OP, (const K*)a.ptr(), na, (const K*)b.ptr(), nb,
                                          (const uint32_t*)nullptr, (const uint32_t*)nullptr, thrust::detail::raw(ko),
                                          (uint32_t*)nullptr, d_num, comp, (hipStream_t)stream);
  throw_on_error(rc, "set operation failed");
  return read_scalar<uint64_t>(d_num, stream, "set operation failed");
}

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
