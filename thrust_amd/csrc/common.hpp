// Shared device-side building blocks for the gfx950 kernels: 16-byte vector access,
// wave64 DPP reductions and scans, the binary-operator set, and the tile-status words
// used by every single-pass (decoupled look-back) kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <type_traits>

#include "../../include/thrust_amd.h"

namespace ta {

constexpr int WAVE = 64;
constexpr int NUM_CU = 256;  // MI355X: 8 XCDs x 32 CUs

#define TA_DEVICE __device__ __forceinline__
#define TA_EXPORT extern "C" __attribute__((visibility("default")))
#define TA_HOST_DEVICE __host__ __device__ __forceinline__

#define TA_CHECK(expr)                         \
  do {                                         \
    hipError_t _e = (expr);                    \
    if (_e != hipSuccess) return (int)_e;      \
  } while (0)

// Launch check that does not clear a sticky error of somebody else.
#define TA_CHECK_LAUNCH() TA_CHECK(hipPeekAtLastError())

TA_HOST_DEVICE size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

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
TA_HOST_DEVICE To bit_cast(const From& f) {
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
TA_DEVICE Vec16<T> load_vec(const T* p) {
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
TA_DEVICE void store_vec(T* p, const Vec16<T>& x) {
  if constexpr (ALIGNED) {
    *reinterpret_cast<Vec16<T>*>(p) = x;
  } else {
#pragma unroll
    for (int i = 0; i < Vec16<T>::N; ++i) p[i] = x.v[i];
  }
}

TA_HOST_DEVICE bool is_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ------------------------------------------------------------------ operators
// Integer addition is done on the unsigned representation so that overflow wraps
// (the reference's int accumulator wraps too; signed overflow would be undefined here).
struct OpPlus {
  template <typename T>
  TA_HOST_DEVICE T operator()(T a, T b) const {
    if constexpr (std::is_integral<T>::value) {
      using U = typename std::make_unsigned<T>::type;
      return (T)(U)((U)a + (U)b);
    } else {
      return a + b;
    }
  }
  // -0.0 is the exact identity of IEEE addition (+0.0 would turn -0.0 into +0.0).
  template <typename T>
  static TA_HOST_DEVICE T identity() {
    if constexpr (std::is_floating_point<T>::value) return (T)-0.0;
    else return (T)0;
  }
};

// a * b in T; integers multiply on the unsigned representation (wraps, no overflow UB).
template <typename T>
TA_DEVICE T mul_wrap(T a, T b) {
  if constexpr (std::is_integral<T>::value && sizeof(T) < 4) {
    // 8- and 16-bit products are made in a 32-bit register of their own; the empty asm
    // keeps them from being packed into byte vectors, which this compiler cannot select
    uint32_t p = (uint32_t)(int32_t)a * (uint32_t)(int32_t)b;
    asm volatile("" : "+v"(p));
    return (T)p;
  } else if constexpr (std::is_integral<T>::value) {
    using U = typename std::make_unsigned<T>::type;
    return (T)(U)((U)a * (U)b);
  } else {
    return a * b;
  }
}

// Unary transforms of the transform_* entry points: thrust::identity, thrust::negate and
// thrust::square (thrust/functional.h:523-600, 1224-1240).  Integers negate and square on
// the unsigned representation (wrap modulo 2^bits).
struct UnIdentity {
  template <typename T>
  TA_DEVICE T operator()(T x) const { return x; }
};
struct UnNegate {
  template <typename T>
  TA_DEVICE T operator()(T x) const {
    if constexpr (std::is_integral<T>::value) {
      using U = typename std::make_unsigned<T>::type;
      return (T)(U)((U)0 - (U)x);
    } else {
      return -x;
    }
  }
};
struct UnSquare {
  template <typename T>
  TA_DEVICE T operator()(T x) const { return mul_wrap(x, x); }
};

template <typename T> struct Limits;
#define TA_LIMITS(T, LO, HI)                                   \
  template <> struct Limits<T> {                               \
    static TA_HOST_DEVICE T lowest() { return LO; }            \
    static TA_HOST_DEVICE T highest() { return HI; }           \
  };
TA_LIMITS(int8_t, INT8_MIN, INT8_MAX)
TA_LIMITS(uint8_t, 0, UINT8_MAX)
TA_LIMITS(int16_t, INT16_MIN, INT16_MAX)
TA_LIMITS(uint16_t, 0, UINT16_MAX)
TA_LIMITS(int32_t, INT32_MIN, INT32_MAX)
TA_LIMITS(uint32_t, 0, UINT32_MAX)
TA_LIMITS(int64_t, INT64_MIN, INT64_MAX)
TA_LIMITS(uint64_t, 0, UINT64_MAX)
TA_LIMITS(float, -__builtin_huge_valf(), __builtin_huge_valf())
TA_LIMITS(double, -__builtin_huge_val(), __builtin_huge_val())
#undef TA_LIMITS

// thrust::minimum: (lhs < rhs) ? lhs : rhs ; thrust::maximum: (lhs < rhs) ? rhs : lhs
// (thrust/functional.h).  Kept in that exact form so NaN / signed-zero behaviour matches.
struct OpMin {
  template <typename T>
  TA_HOST_DEVICE T operator()(T a, T b) const { return (a < b) ? a : b; }
  template <typename T>
  static TA_HOST_DEVICE T identity() { return Limits<T>::highest(); }
};
struct OpMax {
  template <typename T>
  TA_HOST_DEVICE T operator()(T a, T b) const { return (a < b) ? b : a; }
  template <typename T>
  static TA_HOST_DEVICE T identity() { return Limits<T>::lowest(); }
};

// ------------------------------------------------------------------ DPP lane moves
// Moves a value of any size <= 8 bytes one 32-bit half at a time.  Lanes whose source
// is outside the row / wave (or masked off) keep `old`.
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, typename T>
TA_DEVICE T dpp_move(T old, T src) {
  if constexpr (sizeof(T) <= 4) {
    uint32_t o = 0, s = 0;
    __builtin_memcpy(&o, &old, sizeof(T));
    __builtin_memcpy(&s, &src, sizeof(T));
    uint32_t r = (uint32_t)__builtin_amdgcn_update_dpp((int)o, (int)s, CTRL, ROW_MASK, BANK_MASK, false);
    T out;
    __builtin_memcpy(&out, &r, sizeof(T));
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
    __builtin_memcpy(&out, r, sizeof(T));
    return out;
  }
}

template <typename T>
TA_DEVICE T readlane(T v, int lane) {
  if constexpr (sizeof(T) <= 4) {
    uint32_t s = 0;
    __builtin_memcpy(&s, &v, sizeof(T));
    uint32_t r = (uint32_t)__builtin_amdgcn_readlane((int)s, lane);
    T out;
    __builtin_memcpy(&out, &r, sizeof(T));
    return out;
  } else {
    static_assert(sizeof(T) % 4 == 0, "readlane: size must be a multiple of 4 bytes");
    constexpr int WORDS = sizeof(T) / 4;
    uint32_t s[WORDS], r[WORDS];
    __builtin_memcpy(s, &v, sizeof(T));
#pragma unroll
    for (int i = 0; i < WORDS; ++i) r[i] = (uint32_t)__builtin_amdgcn_readlane((int)s[i], lane);
    T out;
    __builtin_memcpy(&out, r, sizeof(T));
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
TA_DEVICE T wave_reduce(T v, Op op) {
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
TA_DEVICE T wave_inclusive_scan(T v, Op op, T id) {
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
TA_DEVICE T wave_inclusive_scan(T v, Op op) {
  return wave_inclusive_scan(v, op, Op::template identity<T>());
}

TA_DEVICE int lane_id() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

// Comparison against a threshold chosen at run time (thrust_amd_cmp codes).
template <int CMP, typename T>
TA_DEVICE bool apply_cmp_code(T x, T t) {
  if constexpr (CMP == THRUST_AMD_LT) return x < t;
  else if constexpr (CMP == THRUST_AMD_LE) return x <= t;
  else if constexpr (CMP == THRUST_AMD_GT) return x > t;
  else if constexpr (CMP == THRUST_AMD_GE) return x >= t;
  else if constexpr (CMP == THRUST_AMD_EQ) return x == t;
  else if constexpr (CMP == THRUST_AMD_NE) return x != t;
  else return x != (T)0;
}

template <typename T>
TA_DEVICE bool apply_cmp(int cmp, T x, T t) {
  const bool negate = (cmp & THRUST_AMD_CMP_NOT) != 0;  // uniform: the logical negation of the code
  bool r;
  switch (cmp & ~THRUST_AMD_CMP_NOT) {
    case THRUST_AMD_LT: r = x < t; break;
    case THRUST_AMD_LE: r = x <= t; break;
    case THRUST_AMD_GT: r = x > t; break;
    case THRUST_AMD_GE: r = x >= t; break;
    case THRUST_AMD_EQ: r = x == t; break;
    case THRUST_AMD_NE: r = x != t; break;
    default: r = x != (T)0; break;
  }
  return r != negate;
}

// Calls f(integral_constant<int, CODE>) for the comparison code inside `cmp` (without its
// negation bit): one uniform branch for a whole tile instead of one per element.
template <typename F>
TA_DEVICE void with_cmp_code(int cmp, F&& f) {
  switch (cmp & ~THRUST_AMD_CMP_NOT) {
    case THRUST_AMD_LT: f(std::integral_constant<int, THRUST_AMD_LT>{}); break;
    case THRUST_AMD_LE: f(std::integral_constant<int, THRUST_AMD_LE>{}); break;
    case THRUST_AMD_GT: f(std::integral_constant<int, THRUST_AMD_GT>{}); break;
    case THRUST_AMD_GE: f(std::integral_constant<int, THRUST_AMD_GE>{}); break;
    case THRUST_AMD_EQ: f(std::integral_constant<int, THRUST_AMD_EQ>{}); break;
    case THRUST_AMD_NE: f(std::integral_constant<int, THRUST_AMD_NE>{}); break;
    default: f(std::integral_constant<int, THRUST_AMD_NONZERO>{}); break;
  }
}

// ------------------------------------------------------------------ search
// First index in [lo, hi] at which a monotone predicate turns false (pred is true on a
// prefix of [lo, hi) and false after it; the result is hi when it is true throughout).
// Plain bisection: for the tile-boundary searches over whole inputs, probing more points
// per round (eight-way per lane, or 64-way per wave) was measured 2x and 5x slower -- the
// lanes of a wave search distant diagonals, every probe is its own cache line and page,
// and the extra probes cost more than the saved rounds.
template <typename Pred>
TA_DEVICE uint64_t partition_point(uint64_t lo, uint64_t hi, Pred pred) {
  while (lo < hi) {
    const uint64_t mid = (lo + hi) >> 1;
    if (pred(mid)) lo = mid + 1;
    else hi = mid;
  }
  return lo;
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
TA_DEVICE void tile_publish(uint64_t* slot, uint32_t status, const P& payload) {
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
TA_DEVICE uint32_t tile_try_load(const uint64_t* slot, P& payload) {
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
  __builtin_memcpy(&payload, words, sizeof(P));
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
template <typename P, typename Op>
TA_DEVICE P tile_lookback(const uint64_t* status_base, uint32_t tile, Op op, P id) {
  constexpr int W = TileWords<P>::W;
  // Descriptors inspected per round: the nearest 8.  A wider window reads more cache lines
  // per round and, with many tiles in flight, costs more than it saves.
  constexpr int WIN = 8;
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

}  // namespace ta
