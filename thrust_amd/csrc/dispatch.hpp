// Run-time (dtype, operator) codes of the C ABI -> compile-time template arguments.
#pragma once
#include "common.hpp"

namespace ta {

inline bool valid_dtype(int d) { return d >= 0 && d < THRUST_AMD_DTYPE_COUNT; }
inline bool valid_binop(int o) { return o >= 0 && o < THRUST_AMD_BINOP_COUNT; }
inline bool valid_cmp(int c) { return c >= 0 && c < THRUST_AMD_CMP_COUNT; }
// ... or its logical negation (the selection entry points accept THRUST_AMD_CMP_NOT)
inline bool valid_cmp_or_not(int c) { return c >= 0 && (c & ~THRUST_AMD_CMP_NOT) < THRUST_AMD_CMP_COUNT; }
inline bool valid_unary(int u) { return u >= 0 && u < THRUST_AMD_UNARY_COUNT; }
inline bool valid_item_bytes(size_t b) { return b == 1 || b == 2 || b == 4 || b == 8; }

template <typename T> struct TypeTag { using type = T; };

// Calls f(TypeTag<T>{}) with the element type of `dtype`.
template <typename F>
inline int with_dtype(int dtype, F&& f) {
  switch (dtype) {
    case THRUST_AMD_I8: return f(TypeTag<int8_t>{});
    case THRUST_AMD_U8: return f(TypeTag<uint8_t>{});
    case THRUST_AMD_I16: return f(TypeTag<int16_t>{});
    case THRUST_AMD_U16: return f(TypeTag<uint16_t>{});
    case THRUST_AMD_I32: return f(TypeTag<int32_t>{});
    case THRUST_AMD_U32: return f(TypeTag<uint32_t>{});
    case THRUST_AMD_I64: return f(TypeTag<int64_t>{});
    case THRUST_AMD_U64: return f(TypeTag<uint64_t>{});
    case THRUST_AMD_F32: return f(TypeTag<float>{});
    case THRUST_AMD_F64: return f(TypeTag<double>{});
    default: return (int)hipErrorInvalidValue;
  }
}

// Calls f(TypeTag<U>{}) with the unsigned integer type of `bytes` bytes (opaque items).
template <typename F>
inline int with_item_bytes(size_t bytes, F&& f) {
  switch (bytes) {
    case 1: return f(TypeTag<uint8_t>{});
    case 2: return f(TypeTag<uint16_t>{});
    case 4: return f(TypeTag<uint32_t>{});
    case 8: return f(TypeTag<uint64_t>{});
    default: return (int)hipErrorInvalidValue;
  }
}

template <typename F>
inline int with_binop(int op, F&& f) {
  switch (op) {
    case THRUST_AMD_PLUS: return f(OpPlus{});
    case THRUST_AMD_MIN: return f(OpMin{});
    case THRUST_AMD_MAX: return f(OpMax{});
    default: return (int)hipErrorInvalidValue;
  }
}

// The transforms other than the identity (callers route the identity to the plain kernels).
template <typename F>
inline int with_transform(int unary, F&& f) {
  switch (unary) {
    case THRUST_AMD_NEGATE: return f(UnNegate{});
    case THRUST_AMD_SQUARE: return f(UnSquare{});
    default: return (int)hipErrorInvalidValue;
  }
}

// Launcher::run<T, Op>(args...) for the (dtype, op) pair.
template <typename Launcher, typename... Args>
inline int dispatch_dtype_op(int dtype, int op, Args... args) {
  return with_dtype(dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_binop(op, [&](auto o) {
      using Op = decltype(o);
      return Launcher::template run<T, Op>(args...);
    });
  });
}

}  // namespace ta
