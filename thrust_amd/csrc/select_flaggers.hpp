// How the selection kernels of the C interface make their flags, shared by the translation
// units that instantiate the compaction kernel (select.hip, select_stencil.hip).
#pragma once
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"

#include "../../include/thrust/system/hip/detail/select_kernels.h"

namespace ta {
using namespace ::thrust::system::hip::select;

// The flags of the C interface: a comparison code and a threshold chosen at run time (one
// uniform branch per tile picks the comparison), the bytes of a flag array, and "differs
// from its predecessor" for unique.
template <typename T>
struct CmpFlagger {
  int cmp;
  T threshold;
  template <typename Body>
  TA_DEVICE void per_tile(Body&& body) const {
    const bool flip = (cmp & THRUST_AMD_CMP_NOT) != 0;
    const T thr = threshold;
    with_cmp_code(cmp, [&](auto code) {
      constexpr int CMP = decltype(code)::value;
      body([thr](const T& x) { return apply_cmp_code<CMP>(x, thr); }, flip);
    });
  }
};
struct ByteFlagger {
  template <typename Body>
  TA_DEVICE void per_tile(Body&& body) const {
    body([](uint8_t x) { return x != 0; }, false);
  }
};
template <typename T>
struct DiffersFlagger {
  template <typename Body>
  TA_DEVICE void per_tile(Body&& body) const {
    body([](const T& before, const T& x) { return !(before == x); }, false);
  }
};

// copy_if / partition_copy by stencil into separate outputs, in one pass (select_stencil.hip).
// Same contract as the entry points: temp == nullptr asks for the size.
int select_by_stencil(void* temp, size_t* temp_bytes, const void* in, const void* stencil, void* out_true,
                      void* out_false, uint64_t* d_num, uint64_t n, size_t item_bytes, int stencil_dtype, int cmp,
                      const void* threshold, hipStream_t stream);

// stable_partition by stencil in place, in one pass (select_stencil_in_place.hip): `data` is both the
// items and where the selected ones end up.
int partition_in_place_by_stencil(void* temp, size_t* temp_bytes, void* data, const void* stencil,
                                  uint64_t* d_num, uint64_t n, size_t item_bytes, int stencil_dtype, int cmp,
                                  const void* threshold, hipStream_t stream);

}  // namespace ta
