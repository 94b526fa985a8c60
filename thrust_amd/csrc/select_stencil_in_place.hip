// The in-place stencil form of thrust_amd_stable_partition: the compaction kernel tests the
// stencil in its own type and moves the items as its payload, sweeping from whichever end
// parks the smaller side -- one pass over stencil and items and the copy back of the parked
// side, no flag array.  What the reference's partition agent does with a stencil
// (thrust/system/cuda/detail/partition.h:796-824).  A translation unit of its own because
// it is two kernels (one per direction) per (stencil type, item size).
#include "select_flaggers.hpp"

namespace ta {

int partition_in_place_by_stencil(void* temp, size_t* temp_bytes, void* data, const void* stencil,
                                  uint64_t* d_num, uint64_t n, size_t item_bytes, int stencil_dtype, int cmp,
                                  const void* threshold, hipStream_t stream) {
  // 256 bytes more than the items: the copy back reads whole 16-byte vectors of the parked items
  const size_t park_bytes = (size_t)n * item_bytes + 256;
  return with_dtype(stencil_dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    const SelectTemp lay = select_layout<T>(n, park_bytes);
    if (!temp) {
      *temp_bytes = lay.total;
      return 0;
    }
    if (*temp_bytes < lay.total || !d_num || (n && (!data || !stencil))) return (int)hipErrorInvalidValue;
    return with_item_bytes(item_bytes, [&](auto ut) {
      using U = typename decltype(ut)::type;
      char* base = static_cast<char*>(temp);
      U* parked = reinterpret_cast<U*>(base + lay.off_extra);
      CmpFlagger<T> flag{};
      flag.cmp = cmp;
      if (threshold) __builtin_memcpy(&flag.threshold, threshold, sizeof(T));
      SelectArgs<T, U, CmpFlagger<T>> a = make_select_args<T, U>(flag);
      a.tested = static_cast<const T*>(stencil);
      a.payload = static_cast<const U*>(data);
      a.payload_true = static_cast<U*>(data);
      a.payload_false = parked;
      a.d_num_true = d_num;
      a.n = n;
      const int rc = select_launch<T, U, FLAG_PRED, true, true, true>(base, lay, a, stream);
      if (rc || n == 0) return rc;
      TA_LAUNCH("partition_tail", stream, (partition_tail_kernel<U>), dim3(tail_grid<U>(n)), dim3(TAIL_BLOCK),
                static_cast<U*>(data), (const U*)parked, n, (const uint64_t*)d_num,
                (const uint32_t*)(reinterpret_cast<uint32_t*>(base + lay.off_ticket) + 16));
      TA_CHECK_LAUNCH();
      return 0;
    });
  });
}

}  // namespace ta
