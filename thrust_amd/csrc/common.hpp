// Shared device-side building blocks for the gfx950 kernels: 16-byte vector access,
// wave64 DPP reductions and scans, the binary-operator set, and the tile-status words
// used by every single-pass (decoupled look-back) kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <type_traits>

#include "../../include/thrust_amd.h"
// launches made by the kernel templates shared with users' translation units go through the
// library's launch wrapper (launch.hpp), so that its per-kernel timing sees them
#define THRUST_AMD_KERNEL_LAUNCH(label, stream, kernel, grid, block, ...) \
  TA_LAUNCH(label, stream, kernel, grid, block, __VA_ARGS__)
#include "../../include/thrust/system/hip/detail/device_primitives.h"

namespace ta {

// vector access, DPP wave operations, OpPlus and the tile-status protocol: shared with the
// kernel templates that users' translation units instantiate
using namespace ::thrust::system::hip::prim;

constexpr int NUM_CU = 256;  // MI355X: 8 XCDs x 32 CUs

#define TA_DEVICE THRUST_AMD_DEVICE
#define TA_EXPORT extern "C" __attribute__((visibility("default")))
#define TA_HOST_DEVICE THRUST_AMD_HOST_DEVICE

#define TA_CHECK(expr)                         \
  do {                                         \
    hipError_t _e = (expr);                    \
    if (_e != hipSuccess) return (int)_e;      \
  } while (0)

// Launch check that does not clear a sticky error of somebody else.
#define TA_CHECK_LAUNCH() TA_CHECK(hipPeekAtLastError())

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

}  // namespace ta
