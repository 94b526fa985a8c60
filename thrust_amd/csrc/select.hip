// thrust_amd_copy_if, thrust_amd_partition_copy, thrust_amd_stable_partition,
// thrust_amd_unique, thrust_amd_unique_by_key: the library's instantiations of the
// single-pass compaction kernel (thrust/system/hip/detail/select_kernels.h describes it)
// for the comparison codes of the C interface.
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"

#include "select_flaggers.hpp"

namespace ta {

// Shared body of copy_if / partition_copy / stable_partition.
//   in_place: out_true == in, rejected elements are parked in temp and moved back.
static int select_by_predicate(void* temp, size_t* temp_bytes, const void* in, const void* stencil,
                               void* out_true, void* out_false, uint64_t* d_num, uint64_t n,
                               size_t item_bytes, int stencil_dtype, int cmp, const void* threshold,
                               bool in_place, hipStream_t stream) {
  if (!temp_bytes || !valid_item_bytes(item_bytes) || !valid_dtype(stencil_dtype) || !valid_cmp_or_not(cmp))
    return (int)hipErrorInvalidValue;
  const size_t tested_bytes = thrust_amd_dtype_size(stencil_dtype);
  if (!stencil && tested_bytes != item_bytes) return (int)hipErrorInvalidValue;
  if ((cmp & ~THRUST_AMD_CMP_NOT) != THRUST_AMD_NONZERO && !threshold && temp) return (int)hipErrorInvalidValue;
  // 256 bytes more than the items: the copy back reads whole 16-byte vectors of the parked items
  const size_t park_bytes = in_place ? (size_t)n * item_bytes + 256 : 0;

  if (!stencil) {
    return with_dtype(stencil_dtype, [&](auto tt) {
      using T = typename decltype(tt)::type;
      const SelectTemp lay = select_layout<T>(n, park_bytes);
      if (!temp) {
        *temp_bytes = lay.total;
        return 0;
      }
      if (*temp_bytes < lay.total || !d_num || (n && (!in || !out_true))) return (int)hipErrorInvalidValue;
      char* base = static_cast<char*>(temp);
      SelectArgs<T, uint32_t, CmpFlagger<T>> a{};
      a.tested = static_cast<const T*>(in);
      a.tested_true = static_cast<T*>(out_true);
      a.tested_false = in_place ? reinterpret_cast<T*>(base + lay.off_extra) : static_cast<T*>(out_false);
      a.d_num_true = d_num;
      a.n = n;
      a.flag.cmp = cmp;
      if (threshold) __builtin_memcpy(&a.flag.threshold, threshold, sizeof(T));
      if (!in_place)
        return a.tested_false ? select_launch<T, uint32_t, FLAG_PRED, false, true>(base, lay, a, stream)
                              : select_launch<T, uint32_t, FLAG_PRED, false>(base, lay, a, stream);
      int rc = select_launch<T, uint32_t, FLAG_PRED, false, true, true>(base, lay, a, stream);
      if (rc || n == 0) return rc;
      TA_LAUNCH("partition_tail", stream, (partition_tail_kernel<T>), dim3(tail_grid<T>(n)), dim3(TAIL_BLOCK),
                static_cast<T*>(out_true), (const T*)(base + lay.off_extra), n, (const uint64_t*)d_num,
                (const uint32_t*)(reinterpret_cast<uint32_t*>(base + lay.off_ticket) + 16));
      TA_CHECK_LAUNCH();
      return 0;
    });
  }
  // stencil form, separate outputs: one pass, the stencil is tested in its own type and the
  // items travel as the payload (select_stencil.hip)
  if (!in_place)
    return select_by_stencil(temp, temp_bytes, in, stencil, out_true, out_false, d_num, n, item_bytes, stencil_dtype,
                             cmp, threshold, stream);
  // stencil form in place: the same one pass, the sweep from whichever end parks the smaller side
  // (select_stencil_in_place.hip)
  return partition_in_place_by_stencil(temp, temp_bytes, out_true, stencil, d_num, n, item_bytes, stencil_dtype, cmp,
                                       threshold, stream);
}

}  // namespace ta

TA_EXPORT int thrust_amd_copy_if(void* temp, size_t* temp_bytes, const void* in, const void* stencil,
                                 void* out, uint64_t* d_num_selected, uint64_t n, size_t item_bytes,
                                 int stencil_dtype, int cmp, const void* threshold, void* stream) {
  return ta::select_by_predicate(temp, temp_bytes, in, stencil, out, nullptr, d_num_selected, n,
                                 item_bytes, stencil_dtype, cmp, threshold, false, (hipStream_t)stream);
}

TA_EXPORT int thrust_amd_partition_copy(void* temp, size_t* temp_bytes, const void* in,
                                        const void* stencil, void* out_true, void* out_false,
                                        uint64_t* d_num_true, uint64_t n, size_t item_bytes,
                                        int stencil_dtype, int cmp, const void* threshold,
                                        void* stream) {
  if (temp && n && !out_false) return (int)hipErrorInvalidValue;
  return ta::select_by_predicate(temp, temp_bytes, in, stencil, out_true, out_false, d_num_true, n,
                                 item_bytes, stencil_dtype, cmp, threshold, false, (hipStream_t)stream);
}

TA_EXPORT int thrust_amd_stable_partition(void* temp, size_t* temp_bytes, void* data,
                                          const void* stencil, uint64_t* d_num_true, uint64_t n,
                                          size_t item_bytes, int stencil_dtype, int cmp,
                                          const void* threshold, void* stream) {
  return ta::select_by_predicate(temp, temp_bytes, data, stencil, data, nullptr, d_num_true, n,
                                 item_bytes, stencil_dtype, cmp, threshold, true, (hipStream_t)stream);
}

TA_EXPORT int thrust_amd_unique_by_key(void* temp, size_t* temp_bytes, const void* keys_in,
                                       const void* values_in, void* keys_out, void* values_out,
                                       uint64_t* d_num_out, uint64_t n, int key_dtype,
                                       size_t value_bytes, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype)) return (int)hipErrorInvalidValue;
  const bool has_values = values_in != nullptr || values_out != nullptr || value_bytes != 0;
  if (has_values && !valid_item_bytes(value_bytes)) return (int)hipErrorInvalidValue;
  return with_dtype(key_dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    const SelectTemp lay = select_layout<T>(n, 0);
    if (!temp) {
      *temp_bytes = lay.total;
      return 0;
    }
    if (*temp_bytes < lay.total || !d_num_out || (n && (!keys_in || !keys_out)))
      return (int)hipErrorInvalidValue;
    if (has_values && n && (!values_in || !values_out)) return (int)hipErrorInvalidValue;
    char* base = static_cast<char*>(temp);
    if (!has_values) {
      SelectArgs<T, uint32_t, DiffersFlagger<T>> a{};
      a.tested = static_cast<const T*>(keys_in);
      a.tested_true = static_cast<T*>(keys_out);
      a.d_num_true = d_num_out;
      a.n = n;
      return select_launch<T, uint32_t, FLAG_HEAD, false>(base, lay, a, (hipStream_t)stream);
    }
    return with_item_bytes(value_bytes, [&](auto ut) {
      using U = typename decltype(ut)::type;
      SelectArgs<T, U, DiffersFlagger<T>> a{};
      a.tested = static_cast<const T*>(keys_in);
      a.payload = static_cast<const U*>(values_in);
      a.tested_true = static_cast<T*>(keys_out);
      a.payload_true = static_cast<U*>(values_out);
      a.d_num_true = d_num_out;
      a.n = n;
      return select_launch<T, U, FLAG_HEAD, true>(base, lay, a, (hipStream_t)stream);
    });
  });
}

TA_EXPORT int thrust_amd_unique(void* temp, size_t* temp_bytes, const void* in, void* out,
                                uint64_t* d_num_out, uint64_t n, int dtype, void* stream) {
  return thrust_amd_unique_by_key(temp, temp_bytes, in, nullptr, out, nullptr, d_num_out, n, dtype, 0,
                                  stream);
}
