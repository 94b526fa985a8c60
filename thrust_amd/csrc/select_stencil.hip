// The stencil forms of thrust_amd_copy_if and thrust_amd_partition_copy: the compaction kernel
// tests the stencil in its own type (comparison code and threshold of the C interface) and
// moves the items as its payload -- one pass, n * (stencil + item) bytes read, no flag array.
// A translation unit of its own because it is one kernel per (stencil type, item size, one or
// two outputs).
#include "select_flaggers.hpp"

namespace ta {

int select_by_stencil(void* temp, size_t* temp_bytes, const void* in, const void* stencil, void* out_true,
                      void* out_false, uint64_t* d_num, uint64_t n, size_t item_bytes, int stencil_dtype, int cmp,
                      const void* threshold, hipStream_t stream) {
  return with_dtype(stencil_dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    const SelectTemp lay = select_layout<T>(n, 0);
    if (!temp) {
      *temp_bytes = lay.total;
      return 0;
    }
    if (*temp_bytes < lay.total || !d_num || (n && (!in || !out_true))) return (int)hipErrorInvalidValue;
    return with_item_bytes(item_bytes, [&](auto ut) {
      using U = typename decltype(ut)::type;
      CmpFlagger<T> flag{};
      flag.cmp = cmp;
      if (threshold) __builtin_memcpy(&flag.threshold, threshold, sizeof(T));
      SelectArgs<T, U, CmpFlagger<T>> a = make_select_args<T, U>(flag);
      a.tested = static_cast<const T*>(stencil);
      a.payload = static_cast<const U*>(in);
      a.payload_true = static_cast<U*>(out_true);
      a.payload_false = static_cast<U*>(out_false);
      a.d_num_true = d_num;
      a.n = n;
      char* base = static_cast<char*>(temp);
      return a.payload_false ? select_launch<T, U, FLAG_PRED, true, true>(base, lay, a, stream)
                             : select_launch<T, U, FLAG_PRED, true>(base, lay, a, stream);
    });
  });
}

}  // namespace ta
