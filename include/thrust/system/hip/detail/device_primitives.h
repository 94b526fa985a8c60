// Device-side building blocks of the gfx950 kernels, shared by the kernels compiled into
// libthrust_amd.so and by the kernel templates that are instantiated in a user's translation
// unit (user predicates, key equalities and operators): 16-byte vector access, wave64 DPP
// reductions and scans, and the tile-status words of the single-pass (decoupled look-back)
// kernels.  HIP code; needs nothing but the HIP runtime.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <type_traits>

#define THRUST_AMD_DEVICE __device__ __forceinline__
#define THRUST_AMD_HOST_DEVICE __host__ __device__ __forceinline__

// Kernel launches of the shared templates go through this macro; the library defines it
// before including them so that its per-kernel timing sees the launches.
#ifndef THRUST_AMD_KERNEL_LAUNCH
#define THRUST_AMD_KERNEL_LAUNCH(label, stream, kernel, grid, block, ...) \
  hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__)
#endif

namespace thrust {
namespace system {
namespace hip {
namespace prim {

constexpr int WAVE = 64;

THRUST_AMD_HOST_DEVICE size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---------------------------------------------------------------- temp carving
// Sub-buffers of a temp allocation, each 256-byte aligned (the reference's
// alias_storage does the same, thrust/system/cuda/detail/core/util.h:752-763).
struct TempLayout {
  size_t total = 0;
  size_t add(size_t bytes) {
    size_t off = total;
    total += align_up(bytes ? bytes : 1, 256);
    return off;
  }
};

// ------------------------------------------------------------------ raw bits
template <int BYTES> struct UIntOf;
template <> struct UIntOf<1> { using type = uint8_t; };
template <> struct UIntOf<2> { using type = uint16_t; };
template <> struct UIntOf<4> { using type = uint32_t; };
template <> struct UIntOf<8> { using type = uint64_t; };
template <typename T> using uint_of_t = typename UIntOf<sizeof(T)>::type;

template <typename To, typename From>
THRUST_AMD_HOST_DEVICE To bit_cast(const From& f) {
  static_assert(sizeof(To) == sizeof(From), "size mismatch");
  return __builtin_bit_cast(To, f);
}

// ------------------------------------------------------------------ 16-byte vectors
template <typename T>
struct alignas(16) Vec16 {
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

// Loads Vec16<T>::N consecutive elements starting at p.  ALIGNED: p is 16-byte aligned
// and one global_load_dwordx4 is emitted; otherwise element-wise loads.
template <bool ALIGNED, typename T>
THRUST_AMD_DEVICE Vec16<T> load_vec(const T* p) {
  if constexpr (ALIGNED) {
    return *reinterpret_cast<const Vec16<T>*>(p);
  } else {
    Vec16<T> r;
#pragma unroll
    for (int i = 0; i < Vec16<T>::N; ++i) r.v[i] = p[i];
    return r;
  }
}

template <bool ALIGNED, typename T>
THRUST_AMD_DEVICE void store_vec(T* p, const Vec16<T>& x) {
  if constexpr (ALIGNED) {
    *reinterpret_cast<Vec16<T>*>(p) = x;
  } else {
#pragma unroll
    for (int i = 0; i < Vec16<T>::N; ++i) p[i] = x.v[i];
  }
}

THRUST_AMD_HOST_DEVICE bool is_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ------------------------------------------------------------------ operators
// Integer addition is done on the unsigned representation so that overflow wraps
// (the reference's int accumulator wraps too; signed overflow would be undefined here).
struct OpPlus {
  template <typename T>
  THRUST_AMD_HOST_DEVICE T operator()(T a, T b) const {
    if constexpr (std::is_integral<T>::value) {
      using U = typename std::make_unsigned<T>::type;
      return (T)(U)((U)a + (U)b);
    } else {
      return a + b;
    }
  }
  // -0.0 is the exact identity of IEEE addition (+0.0 would turn -0.0 into +0.0).
  template <typename T>
  static THRUST_AMD_HOST_DEVICE T identity() {
    if constexpr (std::is_floating_point<T>::value) return (T)-0.0;
    else return (T)0;
  }
};

// ------------------------------------------------------------------ DPP lane moves
// Moves a value of any size <= 8 bytes one 32-bit half at a time.  Lanes whose source
// is outside the row / wave (or masked off) keep `old`.
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, typename T>
THRUST_AMD_DEVICE T dpp_move(T old, T src) {
  if constexpr (sizeof(T) <= 4) {
    uint32_t o = 0, s = 0;
    __builtin_memcpy(&o, (const void*)&old, sizeof(T));
    __builtin_memcpy(&s, (const void*)&src, sizeof(T));
    uint32_t r = (uint32_t)__builtin_amdgcn_update_dpp((int)o, (int)s, CTRL, ROW_MASK, BANK_MASK, false);
    T out;
    __builtin_memcpy((void*)&out, &r, sizeof(T));
    return out;
  } else {
    static_assert(sizeof(T) % 4 == 0, "dpp_move: size must be a multiple of 4 bytes");
    constexpr int WORDS = sizeof(T) / 4;
    uint32_t o[WORDS], s[WORDS], r[WORDS];
    __builtin_memcpy(o, &old, sizeof(T));
    __builtin_memcpy(s, &src, sizeof(T));
#pragma unroll
    for (int i = 0; i < WORDS; ++i)
      r[i] = (uint32_t)__builtin_amdgcn_update_dpp((int)o[i], (int)s[i], CTRL, ROW_MASK, BANK_MASK, false);
    T out;
    __builtin_memcpy((void*)&out, r, sizeof(T));
    return out;
  }
}

template <typename T>
THRUST_AMD_DEVICE T readlane(T v, int lane) {
  if constexpr (sizeof(T) <= 4) {
    uint32_t s = 0;
    __builtin_memcpy(&s, (const void*)&v, sizeof(T));
    uint32_t r = (uint32_t)__builtin_amdgcn_readlane((int)s, lane);
    T out;
    __builtin_memcpy((void*)&out, &r, sizeof(T));
    return out;
  } else {
    static_assert(sizeof(T) % 4 == 0, "readlane: size must be a multiple of 4 bytes");
    constexpr int WORDS = sizeof(T) / 4;
    uint32_t s[WORDS], r[WORDS];
    __builtin_memcpy(s, &v, sizeof(T));
#pragma unroll
    for (int i = 0; i < WORDS; ++i) r[i] = (uint32_t)__builtin_amdgcn_readlane((int)s[i], lane);
    T out;
    __builtin_memcpy((void*)&out, r, sizeof(T));
    return out;
  }
}

// DPP control words (GCN3 / CDNA encoding).
constexpr int DPP_QUAD_XOR1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;
constexpr int DPP_ROW_SHR1 = 0x111, DPP_ROW_SHR2 = 0x112, DPP_ROW_SHR4 = 0x114, DPP_ROW_SHR8 = 0x118;
constexpr int DPP_ROW_BCAST15 = 0x142, DPP_ROW_BCAST31 = 0x143;

// Wave-wide reduction; every lane must be active.  The result is valid in all lanes.
// The combination order is a fixed butterfly inside 16-lane rows, then rows 0..3 left
// to right.
template <typename T, typename Op>
THRUST_AMD_DEVICE T wave_reduce(T v, Op op) {
  v = op(v, dpp_move<DPP_QUAD_XOR1>(v, v));
  v = op(v, dpp_move<DPP_QUAD_XOR2>(v, v));
  v = op(v, dpp_move<DPP_ROW_HALF_MIRROR>(v, v));
  v = op(v, dpp_move<DPP_ROW_MIRROR>(v, v));
  T r0 = readlane(v, 0), r1 = readlane(v, 16), r2 = readlane(v, 32), r3 = readlane(v, 48);
  return op(op(r0, r1), op(r2, r3));
}

// Wave-wide inclusive scan in lane order; every lane must be active.  `id` must be a
// true identity of op (it stands in for lanes that have no left neighbour).
template <typename T, typename Op>
THRUST_AMD_DEVICE T wave_inclusive_scan(T v, Op op, T id) {
  v = op(dpp_move<DPP_ROW_SHR1>(id, v), v);
  v = op(dpp_move<DPP_ROW_SHR2>(id, v), v);
  v = op(dpp_move<DPP_ROW_SHR4>(id, v), v);
  v = op(dpp_move<DPP_ROW_SHR8>(id, v), v);
  // lane 15 of row r -> all lanes of row r+1 (rows 1 and 3), then lane 31 -> rows 2,3
  v = op(dpp_move<DPP_ROW_BCAST15, 0xa>(id, v), v);
  v = op(dpp_move<DPP_ROW_BCAST31, 0xc>(id, v), v);
  return v;
}
template <typename T, typename Op>
THRUST_AMD_DEVICE T wave_inclusive_scan(T v, Op op) {
  return wave_inclusive_scan(v, op, Op::template identity<T>());
}

// A 64-bit value that is the same in every lane of the wave, moved to scalar registers.
THRUST_AMD_DEVICE uint64_t wave_uniform(uint64_t v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}

THRUST_AMD_DEVICE int lane_id() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

// ------------------------------------------------------------------ search
// First index in [lo, hi] at which a monotone predicate turns false (pred is true on a
// prefix of [lo, hi) and false after it; the result is hi when it is true throughout).
// Plain bisection: for the tile-boundary searches over whole inputs, probing more points
// per round (eight-way per lane, or 64-way per wave) was measured 2x and 5x slower -- the
// lanes of a wave search distant diagonals, every probe is its own cache line and page,
// and the extra probes cost more than the saved rounds.
template <typename Pred>
THRUST_AMD_DEVICE uint64_t partition_point(uint64_t lo, uint64_t hi, Pred pred) {
  while (lo < hi) {
    const uint64_t mid = (lo + hi) >> 1;
    if (pred(mid)) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}


// The same search, probing at every step the index of its interval that is a multiple of the
// largest power of two.  It needs as many steps as the bisection at worst, but the probes of the
// first steps are the same few indices for every thread that searches the same arrays (the
// nodes of one implicit tree over the index range), so they come from the caches instead of
// each being a miss of its own: the searches for the tile boundaries of a merge of 2 x 2^27 keys
// (65537 threads, 27 dependent steps each) took 108 us with the plain bisection.
template <typename Pred>
THRUST_AMD_DEVICE uint64_t aligned_partition_point(uint64_t lo, uint64_t hi, Pred pred) {
  while (lo < hi) {
    const uint64_t last = hi - 1;
    const uint64_t differ = lo ^ last;
    const uint64_t mid = differ ? (last & ~((1ull << (63 - __builtin_clzll(differ))) - 1ull)) : lo;
    if (pred(mid)) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

// The same partition point, for a caller that knows an index `from` (lo <= from <= hi) near it: steps of
// doubling length away from `from` bracket the point, a bisection inside the bracket finds it.  The
// number of probes grows with the logarithm of the distance, not of the range.
template <typename Pred>
THRUST_AMD_DEVICE uint64_t nearby_partition_point(uint64_t lo, uint64_t hi, uint64_t from, Pred pred) {
  from = from < lo ? lo : (from > hi ? hi : from);
  uint64_t l, r;
  if (from < hi && pred(from)) {  // the point lies after `from`
    l = from + 1;
    r = hi;
    for (uint64_t step = 1;; step <<= 1) {
      if (hi - l < step) break;  // the probe would be hi or later
      const uint64_t probe = l + step - 1;
      if (pred(probe)) {
        l = probe + 1;
      } else {
        r = probe;
        break;
      }
    }
  } else {  // the point lies at or before `from`
    l = lo;
    r = from;
    for (uint64_t step = 1;; step <<= 1) {
      if (r - lo < step) break;  // the probe would lie before lo
      const uint64_t probe = r - step;
      if (!pred(probe)) {
        r = probe;
      } else {
        l = probe + 1;
        break;
      }
    }
  }
  while (l < r) {
    const uint64_t mid = l + ((r - l) >> 1);
    if (pred(mid)) l = mid + 1;
    else r = mid;
  }
  return l;
}

// The element at an address of global memory that was computed as an integer (the compiler
// cannot tell where such an address points and would use the slower generic load).  Elements
// of the usual sizes travel as one integer of their size; E is trivially copyable.
template <typename E>
THRUST_AMD_DEVICE E load_global(uintptr_t address) {
  if constexpr ((sizeof(E) == 1 || sizeof(E) == 2 || sizeof(E) == 4 || sizeof(E) == 8) && alignof(E) >= sizeof(E)) {
    using Raw = std::conditional_t<sizeof(E) == 1, uint8_t,
                                   std::conditional_t<sizeof(E) == 2, uint16_t,
                                                      std::conditional_t<sizeof(E) == 4, uint32_t, uint64_t>>>;
    typedef const Raw __attribute__((address_space(1))) * in_global_memory;
    const Raw raw = *reinterpret_cast<in_global_memory>(address);
    E e;
    __builtin_memcpy(&e, &raw, sizeof(E));
    return e;
  } else {
    return *reinterpret_cast<const E*>(address);
  }
}

// ------------------------------------------------------------------ merging inside a tile
// A tile of a merge holds two sorted parts side by side in LDS: s[0, ca) from the first range and
// s[ca, count) from the second.  (The set operations use these; the merge and merge sort kernels
// keep their own predicated staging, which measured faster for them with 8-byte keys and values.)

// Stages the tile: element e of the tile is pa[e] for e < ca and pb[e - ca] after that; thread t
// loads the elements t, t + BLOCK, ...  Slots from `count` up to BLOCK * ITEMS receive a copy of
// the tile's last element (count >= 1), so that every slot holds a value of the input.
template <int BLOCK, int ITEMS, typename E>
THRUST_AMD_DEVICE void stage_two_parts(const E* __restrict__ pa, const E* __restrict__ pb, uint32_t ca, uint32_t count,
                                       E* s) {
  E in[ITEMS];
  if (count == (uint32_t)BLOCK * ITEMS) {
    // A full tile.  The 64 elements a wave loads per step are consecutive, so all but at most one
    // of its steps lie inside one part: there the address is a base that is the same for the
    // whole wave (scalar arithmetic) plus the lane's offset, and nothing is computed per lane.
    // The caller's arguments are the same in every lane; saying so keeps them in scalar registers.
    const uint32_t lane = threadIdx.x % WAVE;
    const uint32_t first = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x - lane));
    const uint32_t ca_u = (uint32_t)__builtin_amdgcn_readfirstlane((int)ca);
    const uintptr_t base_a = wave_uniform(reinterpret_cast<uintptr_t>(pa)) + (uintptr_t)first * sizeof(E);
    const uintptr_t base_b = wave_uniform(reinterpret_cast<uintptr_t>(pb)) +
                             (uintptr_t)(((intptr_t)first - (intptr_t)ca_u) * (intptr_t)sizeof(E));
    const uint32_t off = lane * (uint32_t)sizeof(E);
#pragma unroll
    for (int q = 0; q < ITEMS; ++q) {
      const int32_t lanes_of_a = (int32_t)ca_u - (int32_t)((uint32_t)q * BLOCK + first);
      const uintptr_t step = (uintptr_t)q * BLOCK * sizeof(E);
      if (lanes_of_a >= WAVE) in[q] = load_global<E>(base_a + step + off);
      else if (lanes_of_a <= 0) in[q] = load_global<E>(base_b + step + off);
      else in[q] = load_global<E>(((int32_t)lane < lanes_of_a ? base_a : base_b) + step + off);
    }
  } else {
    // (the arithmetic stays on pointers so that the loads are known to go to global memory)
    const E* const base_b = pb - ca;  // only indexed from ca on
#pragma unroll
    for (int q = 0; q < ITEMS; ++q) {
      uint32_t e = (uint32_t)q * BLOCK + threadIdx.x;
      e = e < count ? e : count - 1;
      in[q] = (e < ca ? pa : base_b)[e];
    }
  }
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) s[(uint32_t)q * BLOCK + threadIdx.x] = in[q];
}

// Number of elements of the first part among the first `diag` elements of the merged order
// (an element of the second part is taken only when it is before the first part's: ties go to the first).
template <typename T, typename Comp>
THRUST_AMD_DEVICE uint32_t merge_path_in_tile(const T* s, uint32_t ca, uint32_t count, uint32_t diag, Comp& comp) {
  const uint32_t cb = count - ca;
  uint32_t lo = diag > cb ? diag - cb : 0u, hi = diag < ca ? diag : ca;
  while (lo < hi) {
    const uint32_t mid = (lo + hi) >> 1;
    if (!comp(s[ca + diag - 1 - mid], s[mid])) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

// ITEMS steps of the merge from slot i of the first part and slot j of the second (i + j - ca elements
// are already merged).  emit(o, element, slot, from_second) receives the steps in order.  The
// comparator only sees elements of the parts (candidates past their ends are not compared); slots
// read stay at or below count + ITEMS.
template <int ITEMS, typename T, typename Comp, typename Emit>
THRUST_AMD_DEVICE void merge_steps(const T* s, uint32_t i, uint32_t j, uint32_t ca, uint32_t count, Comp& comp,
                                   Emit emit) {
  T ka = s[i], kb = s[j];
#pragma unroll
  for (int o = 0; o < ITEMS; ++o) {
    const bool take_b = (j < count) && (i >= ca || comp(kb, ka));
    emit(o, take_b ? kb : ka, take_b ? j : i, take_b);
    const uint32_t next = take_b ? ++j : ++i;
    const T nk = s[next];
    if (take_b) kb = nk;
    else ka = nk;
  }
}

// ------------------------------------------------------------------ tile status
// A tile publishes W 32-bit payload words, each inside its own 64-bit word together
// with the status, using relaxed agent-scope atomics.  A reader accepts a descriptor
// only when all W words carry the same non-zero status; every status value is written
// at most once per tile, so equal statuses imply the words belong together.  No fence
// is needed because nothing but the descriptor itself is communicated.
enum : uint32_t { TS_INVALID = 0, TS_PARTIAL = 1, TS_INCLUSIVE = 2 };

template <typename P>
struct TileWords {
  static constexpr int W = (sizeof(P) + 3) / 4;
};

template <typename P>
THRUST_AMD_DEVICE void tile_publish(uint64_t* slot, uint32_t status, const P& payload) {
  constexpr int W = TileWords<P>::W;
  uint32_t words[W] = {};
  __builtin_memcpy(words, &payload, sizeof(P));
#pragma unroll
  for (int i = 0; i < W; ++i) {
    __hip_atomic_store(slot + i, ((uint64_t)status << 32) | words[i], __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Returns the status (TS_INVALID when the descriptor is not ready or torn).
template <typename P>
THRUST_AMD_DEVICE uint32_t tile_try_load(const uint64_t* slot, P& payload) {
  constexpr int W = TileWords<P>::W;
  uint32_t words[W];
  uint32_t status = 0;
  bool same = true;
#pragma unroll
  for (int i = 0; i < W; ++i) {
    uint64_t x = __hip_atomic_load(slot + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t s = (uint32_t)(x >> 32);
    words[i] = (uint32_t)x;
    if (i == 0) status = s;
    else same = same && (s == status);
  }
  __builtin_memcpy((void*)&payload, words, sizeof(P));
  return same ? status : (uint32_t)TS_INVALID;
}

// Decoupled look-back run by one full wave (all 64 lanes active, uniform control flow).
// Tile `tile` (> 0) has already published its own PARTIAL descriptor.  In each round
// lane l of the highest WIN lanes inspects tile (base - 63 + l), so lane order equals tile
// order and lane 63 is the nearest predecessor; the wave folds, oldest to newest, everything from the
// nearest INCLUSIVE descriptor up to tile - 1.  Only tiles with a smaller ticket are
// waited on, and those have started, so the spin terminates without assuming any
// workgroup scheduling order.  `id` must be a true identity of op.  Returns, in all
// lanes, the fold of all tiles before `tile`.
template <typename P, int WINDOW = 8, typename Op>
THRUST_AMD_DEVICE P tile_lookback(const uint64_t* status_base, uint32_t tile, Op op, P id) {
  constexpr int W = TileWords<P>::W;
  // Descriptors inspected per round: the nearest WINDOW.  A wider window reads more cache lines
  // per round and, with many tiles in flight, mostly costs more than it saves: 8 measured best
  // for the scans and the selection kernels, 16 for reduce_by_key (whose tiles have little left
  // to do once their prefix is known: 0.617 -> 0.600 ms at 2^28 pairs).
  constexpr int WIN = WINDOW;
  const int lane = lane_id();
  P running = id;
  int64_t base = (int64_t)tile - 1;
  for (;;) {
    const int64_t idx = base - 63 + lane;
    P val = id;
    uint32_t st;
    uint64_t needed;
    for (;;) {
      if (lane < WAVE - WIN) {
        st = TS_PARTIAL;  // outside the window: contributes nothing
        val = id;
      } else if (idx >= 0) {
        st = tile_try_load<P>(status_base + (size_t)idx * W, val);
      } else {
        st = TS_INCLUSIVE;  // before tile 0: an inclusive prefix that contributes nothing
        val = id;
      }
      const uint64_t invalid = __builtin_amdgcn_ballot_w64(st == TS_INVALID);
      const uint64_t incl = __builtin_amdgcn_ballot_w64(st == TS_INCLUSIVE);
      // lanes from the nearest (highest-lane) inclusive descriptor upwards
      needed = incl ? (~0ull << (63 - __builtin_clzll(incl))) : ~0ull;
      if ((invalid & needed) == 0) {
        const bool found = incl != 0;
        const P contrib = ((needed >> lane) & 1) ? val : id;
        const P window = readlane(wave_inclusive_scan(contrib, op, id), 63);
        running = op(window, running);
        if (found) return running;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    base -= WIN;
  }
}
}  // namespace prim
}  // namespace hip
}  // namespace system
}  // namespace thrust
