// copy_if, remove_if, the partition family, unique and unique_by_key for a user's predicate,
// key equality or element struct (hipcc translation units): the library's single-pass
// compaction kernel, instantiated here with the functor inside it, as the reference passes
// the functor into its agents (thrust/system/cuda/detail/copy_if.h:547-556,
// partition.h:221-293, unique.h:316-445, unique_by_key.h:348-510).  One pass over the input
// and no flag array: the predicate runs on the elements in registers.
//
// What is tested (the elements themselves, a stencil, or keys for their run beginnings) is
// read as its own type, 1, 2, 4, 8 or 16 bytes wide; what is moved besides travels as opaque
// items of 1, 2, 4 or 8 bytes.
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/hip/detail/generic_select.h is HIP code: compile this translation unit with hipcc"
#endif
#include <type_traits>

#include <thrust/pair.h>
#include <thrust/tuple.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/select_kernels.h>

namespace thrust {
namespace system {
namespace hip {
namespace detail {

// flag = pred(x), inverted for the remove family
template <typename Pred>
struct pred_flagger {
  mutable Pred pred;
  bool negate;
  template <typename Body>
  __device__ __forceinline__ void per_tile(Body&& body) const {
    body([this](const auto& x) -> bool { return pred(x); }, negate);
  }
};
// head flag = the key does not continue its predecessor's run
template <typename Eq>
struct run_flagger {
  mutable Eq eq;
  template <typename Body>
  __device__ __forceinline__ void per_tile(Body&& body) const {
    body([this](const auto& before, const auto& x) -> bool { return !eq(before, x); }, false);
  }
};

// What the kernel can hold in registers and load as (parts of) 16-byte vectors.  Trivially
// copyable in full: the kernel assigns elements to registers and to staging memory that no
// constructor has run on, which a type with an assignment operator of its own may not survive
// (such a type has its predicate evaluated into flags first and is then moved as bytes).
// A thrust::tuple or thrust::pair of such values counts: its assignment operator is its own (a
// tuple of references assigns through) but assigns member by member, which is the same bytes.
template <typename S>
struct is_bytewise_copyable : std::is_trivially_copyable<S> {};
template <>
struct is_bytewise_copyable<thrust::tuple<> > : std::true_type {};
template <typename H, typename... T>
struct is_bytewise_copyable<thrust::tuple<H, T...> >
    : std::integral_constant<bool, !std::is_reference<H>::value && is_bytewise_copyable<H>::value &&
                                       is_bytewise_copyable<thrust::tuple<T...> >::value> {};
template <typename A, typename B>
struct is_bytewise_copyable<thrust::pair<A, B> >
    : std::integral_constant<bool, !std::is_reference<A>::value && !std::is_reference<B>::value &&
                                       is_bytewise_copyable<A>::value && is_bytewise_copyable<B>::value> {};
template <typename S>
struct is_kernel_item
    : std::integral_constant<bool, is_bytewise_copyable<S>::value && std::is_default_constructible<S>::value &&
                                       (sizeof(S) == 1 || sizeof(S) == 2 || sizeof(S) == 4 || sizeof(S) == 8 ||
                                        sizeof(S) == 16) &&
                                       (alignof(S) <= 16)> {};

namespace select_detail {
namespace sel = ::thrust::system::hip::select;

struct carved_temp {
  char* base;
  uint64_t* d_num;
  sel::SelectTemp lay;
};
template <typename Tested>
inline carved_temp carve(temp_storage& temp, uint64_t n, std::size_t extra_bytes) {
  carved_temp c;
  c.lay = sel::select_layout<Tested>(n, extra_bytes);
  temp.ensure(c.lay.total + 256);
  c.base = static_cast<char*>(temp.ptr());
  c.d_num = reinterpret_cast<uint64_t*>(c.base + c.lay.total);
  return c;
}
template <typename U>
inline int move_parked_back(const carved_temp& c, U* data, uint64_t n, hipStream_t stream) {
  THRUST_AMD_KERNEL_LAUNCH("partition_tail", stream, (sel::partition_tail_kernel<U>), dim3(sel::tail_grid<U>(n)),
                           dim3(sel::TAIL_BLOCK), data, (const U*)(c.base + c.lay.off_extra), n,
                           (const uint64_t*)c.d_num,
                           (const uint32_t*)(reinterpret_cast<uint32_t*>(c.base + c.lay.off_ticket) + 16));
  return (int)hipPeekAtLastError();
}
}  // namespace select_detail

// The selection by a predicate in all its shapes; returns how many elements it selected.
//   stencil    what the predicate sees (HAS_STENCIL), else the items themselves
//   out_false  where the rejected items go (partition_copy), or null
//   in_place   stable_partition: out_true == items, the smaller side is parked in temporary
//              storage during the sweep and copied back
// out_true may be the items themselves for the forward compaction (remove_if): an element
// never lands behind its source, and a tile is written only after every earlier one was read.
template <bool HAS_STENCIL, typename T, typename S, typename Pred>
uint64_t generic_selection(void* stream, const temp_source& source, const T* items, const S* stencil, T* out_true,
                           T* out_false, bool in_place, uint64_t n, const Pred& pred, bool negate, const char* what) {
  namespace sel = ::thrust::system::hip::select;
  typedef pred_flagger<Pred> F;
  typedef typename sel::UIntOf<sizeof(T)>::type U;
  typedef typename std::conditional<HAS_STENCIL, S, T>::type Tested;
  static_assert(is_kernel_item<Tested>::value,
                "selection with a user's predicate: the tested type must be trivially copyable, 1, 2, 4, 8 or 16 bytes");
  hipStream_t s = (hipStream_t)stream;
  temp_storage temp(stream, source);
  const std::size_t park_bytes = in_place ? (std::size_t)n * sizeof(T) + 256 : 0;
  const select_detail::carved_temp c = select_detail::carve<Tested>(temp, n, park_bytes);
  sel::SelectArgs<Tested, U, F> a = sel::make_select_args<Tested, U>(F{pred, negate});
  a.d_num_true = c.d_num;
  a.n = n;
  int rc;
  if constexpr (!HAS_STENCIL) {
    a.tested = reinterpret_cast<const Tested*>(items);
    a.tested_true = reinterpret_cast<Tested*>(out_true);
    a.tested_false = in_place ? reinterpret_cast<Tested*>(c.base + c.lay.off_extra) : reinterpret_cast<Tested*>(out_false);
    if (in_place) {
      rc = sel::select_launch<Tested, U, sel::FLAG_PRED, false, true, true>(c.base, c.lay, a, s);
      if (rc == 0) rc = select_detail::move_parked_back<Tested>(c, reinterpret_cast<Tested*>(out_true), n, s);
    } else if (out_false) {
      rc = sel::select_launch<Tested, U, sel::FLAG_PRED, false, true>(c.base, c.lay, a, s);
    } else {
      rc = sel::select_launch<Tested, U, sel::FLAG_PRED, false>(c.base, c.lay, a, s);
    }
  } else {
    a.tested = stencil;
    a.payload = reinterpret_cast<const U*>(items);
    a.payload_true = reinterpret_cast<U*>(out_true);
    a.payload_false = in_place ? reinterpret_cast<U*>(c.base + c.lay.off_extra) : reinterpret_cast<U*>(out_false);
    if (in_place) {
      rc = sel::select_launch<Tested, U, sel::FLAG_PRED, true, true, true>(c.base, c.lay, a, s);
      if (rc == 0) rc = select_detail::move_parked_back<U>(c, reinterpret_cast<U*>(out_true), n, s);
    } else if (out_false) {
      rc = sel::select_launch<Tested, U, sel::FLAG_PRED, true, true>(c.base, c.lay, a, s);
    } else {
      rc = sel::select_launch<Tested, U, sel::FLAG_PRED, true>(c.base, c.lay, a, s);
    }
  }
  throw_on_error(rc, what);
  return read_scalar<uint64_t>(c.d_num, stream, what);
}

// The first key (and value) of every run of keys that eq() chains together; returns the
// number of runs.  The outputs may be the inputs.
template <typename K, typename Eq>
uint64_t generic_unique(void* stream, const temp_source& source, const K* keys, K* keys_out, uint64_t n, const Eq& eq,
                        const char* what) {
  namespace sel = ::thrust::system::hip::select;
  typedef run_flagger<Eq> F;
  static_assert(is_kernel_item<K>::value,
                "unique with a user's predicate: elements must be trivially copyable, 1, 2, 4, 8 or 16 bytes");
  temp_storage temp(stream, source);
  const select_detail::carved_temp c = select_detail::carve<K>(temp, n, 0);
  sel::SelectArgs<K, uint32_t, F> a = sel::make_select_args<K, uint32_t>(F{eq});
  a.tested = keys;
  a.tested_true = keys_out;
  a.d_num_true = c.d_num;
  a.n = n;
  throw_on_error(sel::select_launch<K, uint32_t, sel::FLAG_HEAD, false>(c.base, c.lay, a, (hipStream_t)stream), what);
  return read_scalar<uint64_t>(c.d_num, stream, what);
}
template <typename K, typename V, typename Eq>
uint64_t generic_unique_by_key(void* stream, const temp_source& source, const K* keys, const V* values, K* keys_out,
                               V* values_out, uint64_t n, const Eq& eq, const char* what) {
  namespace sel = ::thrust::system::hip::select;
  typedef run_flagger<Eq> F;
  typedef typename sel::UIntOf<sizeof(V)>::type U;
  static_assert(is_kernel_item<K>::value,
                "unique_by_key with a user's predicate: keys must be trivially copyable, 1, 2, 4, 8 or 16 bytes");
  temp_storage temp(stream, source);
  const select_detail::carved_temp c = select_detail::carve<K>(temp, n, 0);
  sel::SelectArgs<K, U, F> a = sel::make_select_args<K, U>(F{eq});
  a.tested = keys;
  a.payload = reinterpret_cast<const U*>(values);
  a.tested_true = keys_out;
  a.payload_true = reinterpret_cast<U*>(values_out);
  a.d_num_true = c.d_num;
  a.n = n;
  throw_on_error(sel::select_launch<K, U, sel::FLAG_HEAD, true>(c.base, c.lay, a, (hipStream_t)stream), what);
  return read_scalar<uint64_t>(c.d_num, stream, what);
}

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
