// Glue between the templated front end and the C ABI of libthrust_amd:
//   - element types -> dtype codes, functor types -> operator codes (compile time);
//     an unsupported combination is a static_assert naming the limitation, the analogue
//     of the reference's "unimplemented for this system" terminals
//     (thrust/system/detail/generic/reduce.inl:56-72),
//   - temp_storage: RAII over the temp arena (the reference allocates a
//     temporary_array<uint8_t,Derived>, thrust/system/cuda/detail/reduce.h:959-960),
//   - run(): the two-phase size-query / run protocol plus error conversion.
#pragma once
#include <cstdint>
#include <cmath>
#include <limits>
#include <type_traits>

#include <thrust/detail/execution_policy.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/iterator/iterator_traits.h>
#include <thrust/system_error.h>
#include <thrust_amd.h>

namespace thrust {
namespace system {
namespace hip {
namespace detail {

template <typename T, typename Enable = void>
struct dtype_of { static const int value = -1; };
template <typename T>
struct dtype_of<T, typename std::enable_if<std::is_integral<T>::value && !std::is_same<T, bool>::value>::type> {
  static const int value = sizeof(T) == 1 ? (std::is_signed<T>::value ? THRUST_AMD_I8 : THRUST_AMD_U8)
                         : sizeof(T) == 2 ? (std::is_signed<T>::value ? THRUST_AMD_I16 : THRUST_AMD_U16)
                         : sizeof(T) == 4 ? (std::is_signed<T>::value ? THRUST_AMD_I32 : THRUST_AMD_U32)
                                          : (std::is_signed<T>::value ? THRUST_AMD_I64 : THRUST_AMD_U64);
};
template <> struct dtype_of<float> { static const int value = THRUST_AMD_F32; };
template <> struct dtype_of<double> { static const int value = THRUST_AMD_F64; };

template <typename T>
struct is_abi_type : std::integral_constant<bool, (dtype_of<T>::value >= 0)> {};
// Moved as bytes: copying the object representation is copy construction, and nothing needs to
// run when a copy goes away.  (The type may still define an assignment of its own; elements
// are never assigned to, only constructed from bytes.)
template <typename T>
struct is_bytewise_movable : std::integral_constant<bool, std::is_trivially_copy_constructible<T>::value &&
                                                          std::is_trivially_destructible<T>::value> {};
template <typename T>
struct is_abi_item : std::integral_constant<bool, is_bytewise_movable<T>::value &&
                                                  (sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8)> {};

// ---- functor types -> codes
template <typename Op, typename T> struct binop_code { static const int value = -1; };
template <typename T> struct binop_code<thrust::plus<T>, T> { static const int value = THRUST_AMD_PLUS; };
template <typename T> struct binop_code<thrust::plus<void>, T> { static const int value = THRUST_AMD_PLUS; };
template <typename T> struct binop_code<thrust::minimum<T>, T> { static const int value = THRUST_AMD_MIN; };
template <typename T> struct binop_code<thrust::minimum<void>, T> { static const int value = THRUST_AMD_MIN; };
template <typename T> struct binop_code<thrust::maximum<T>, T> { static const int value = THRUST_AMD_MAX; };
template <typename T> struct binop_code<thrust::maximum<void>, T> { static const int value = THRUST_AMD_MAX; };

// thrust_amd_unary code of a transform whose argument and result are T, or -1
template <typename Fn, typename T> struct unary_code { static const int value = -1; };
template <typename T> struct unary_code<thrust::identity<T>, T> { static const int value = THRUST_AMD_IDENTITY; };
template <typename T> struct unary_code<thrust::identity<void>, T> { static const int value = THRUST_AMD_IDENTITY; };
template <typename T> struct unary_code<thrust::negate<T>, T> { static const int value = THRUST_AMD_NEGATE; };
template <typename T> struct unary_code<thrust::negate<void>, T> { static const int value = THRUST_AMD_NEGATE; };
template <typename T> struct unary_code<thrust::square<T>, T> { static const int value = THRUST_AMD_SQUARE; };
template <typename T> struct unary_code<thrust::square<void>, T> { static const int value = THRUST_AMD_SQUARE; };

// 0 ascending (less), 1 descending (greater), -1 not a recognised ordering
template <typename Comp, typename T> struct order_code { static const int value = -1; };
template <typename T> struct order_code<thrust::less<T>, T> { static const int value = 0; };
template <typename T> struct order_code<thrust::less<void>, T> { static const int value = 0; };
template <typename T> struct order_code<thrust::greater<T>, T> { static const int value = 1; };
template <typename T> struct order_code<thrust::greater<void>, T> { static const int value = 1; };

template <typename Pred, typename T> struct is_equal_to : std::false_type {};
template <typename T> struct is_equal_to<thrust::equal_to<T>, T> : std::true_type {};
template <typename T> struct is_equal_to<thrust::equal_to<void>, T> : std::true_type {};

// Unary predicate -> (cmp code, threshold of the tested type).
template <typename Pred, typename T>
struct unary_pred {
  static const bool supported = false;
  static int cmp(const Pred&) { return -1; }
  static T threshold(const Pred&) { return T(); }
};
// `x CMP t` with a threshold of type U on elements of type T.  C++ evaluates it after the usual
// arithmetic conversions; the kernel compares two values of type T.  The two agree in three
// situations, told apart by the types:
//   SAME        converting t to T is the very conversion C++ applies (or loses nothing)
//   MATH_INT    C++ compares the mathematical values of two integers: a threshold inside T's
//               range is cast, one outside it makes the predicate constant
//   MATH_FLOAT  integer elements against a floating threshold that every element converts to
//               exactly: `x < 2.5` is `x < 3`, `x == 2.5` is never true
// Every other combination (float elements against a double threshold, signed elements
// converted to unsigned, ...) is not evaluated in the kernel; the caller's predicate is then
// applied as it stands by a kernel instantiated for it.
template <int CMP, typename U, typename T>
struct unary_pred<thrust::detail::compare_with<CMP, U>, T> {
  enum kind_t { NONE, SAME, MATH_INT, MATH_UINT, MATH_FLOAT };
  template <typename A, typename B, bool = std::is_arithmetic<A>::value && std::is_arithmetic<B>::value>
  struct classify { static const int value = NONE; };
  template <typename A, typename B>
  struct classify<A, B, true> {
    typedef typename std::common_type<decltype(+A()), decltype(+B())>::type C;  // after promotion
    static const bool a_f = std::is_floating_point<A>::value, b_f = std::is_floating_point<B>::value;
    static const int value =
        a_f ? ((!b_f || sizeof(B) <= sizeof(A)) ? SAME : NONE)
        : b_f ? (((std::is_same<B, double>::value && sizeof(A) <= 4) || (std::is_same<B, float>::value && sizeof(A) <= 2))
                     ? MATH_FLOAT : NONE)
        : std::is_signed<C>::value ? MATH_INT
        : std::is_unsigned<A>::value ? MATH_UINT
                                     : NONE;
  };
  static const int kind = classify<T, U>::value;
  static const bool supported = kind != NONE;

  struct resolved { int cmp; T thr; };
  static resolved constant(bool always) {
    // always true: x >= lowest; always false: x < lowest
    return resolved{always ? THRUST_AMD_GE : THRUST_AMD_LT, std::numeric_limits<T>::lowest()};
  }
  // x CMP w for x over T's whole range, w a wide integer of type Wide
  template <typename Wide>
  static resolved against_integer(int cmp, Wide w) {
    const Wide lo = (Wide)std::numeric_limits<T>::lowest(), hi = (Wide)std::numeric_limits<T>::max();
    if (w >= lo && w <= hi) return resolved{cmp, (T)w};
    const bool above = w > hi;  // every element is below (above) the threshold
    switch (cmp) {
      case THRUST_AMD_LT: case THRUST_AMD_LE: return constant(above);
      case THRUST_AMD_GT: case THRUST_AMD_GE: return constant(!above);
      case THRUST_AMD_EQ: return constant(false);
      default: return constant(true);
    }
  }
  static resolved resolve(const thrust::detail::compare_with<CMP, U>& p, std::integral_constant<int, SAME>) {
    return resolved{CMP, static_cast<T>(p.value)};
  }
  static resolved resolve(const thrust::detail::compare_with<CMP, U>& p, std::integral_constant<int, MATH_INT>) {
    return against_integer<long long>(CMP, (long long)p.value);
  }
  static resolved resolve(const thrust::detail::compare_with<CMP, U>& p, std::integral_constant<int, MATH_UINT>) {
    typedef typename classify<T, U>::C C;  // the threshold wraps to C, as in C++; elements keep their value
    return against_integer<unsigned long long>(CMP, (unsigned long long)(C)p.value);
  }
  static resolved resolve(const thrust::detail::compare_with<CMP, U>& p, std::integral_constant<int, MATH_FLOAT>) {
    const double v = (double)p.value;
    if (v != v) return constant(CMP == THRUST_AMD_NE);  // NaN
    const double fl = std::floor(v), ce = std::ceil(v);
    const bool whole = fl == v;
    int cmp = CMP;
    double w = v;
    switch (CMP) {
      case THRUST_AMD_LT: case THRUST_AMD_GE: w = ce; break;
      case THRUST_AMD_LE: case THRUST_AMD_GT: w = fl; break;
      default: if (!whole) return constant(CMP == THRUST_AMD_NE); break;
    }
    // T has at most 32 bits here: anything beyond +-2^62 is outside its range on that side
    const long long wide = w >= 4.0e18 ? (1LL << 62) : (w <= -4.0e18 ? -(1LL << 62) : (long long)w);
    return against_integer<long long>(cmp, wide);
  }
  static resolved resolve(const thrust::detail::compare_with<CMP, U>&, std::integral_constant<int, NONE>) {
    return resolved{-1, T()};
  }
  static int cmp(const thrust::detail::compare_with<CMP, U>& p) { return resolve(p, std::integral_constant<int, kind>()).cmp; }
  static T threshold(const thrust::detail::compare_with<CMP, U>& p) { return resolve(p, std::integral_constant<int, kind>()).thr; }
};
template <typename I, typename T>
struct unary_pred<thrust::identity<I>, T> {
  static const bool supported = true;
  static int cmp(const thrust::identity<I>&) { return THRUST_AMD_NONZERO; }
  static T threshold(const thrust::identity<I>&) { return T(); }
};
template <typename I, typename T>
struct unary_pred<thrust::logical_not<I>, T> {
  static const bool supported = true;
  static int cmp(const thrust::logical_not<I>&) { return THRUST_AMD_EQ; }
  static T threshold(const thrust::logical_not<I>&) { return T(0); }
};

// ---- temp storage, returned when the scope ends: from the library's arena, or from the
// allocator of a par(alloc) policy.  A user allocator may hand out memory of any
// alignment, so 256 more bytes are requested and the pointer is rounded up; its memory
// goes back only after the stream has drained (the arena's release is stream-ordered).
class temp_storage {
 public:
  temp_storage(void* stream, const temp_source& source)
      : ptr_(nullptr), raw_(nullptr), stream_(stream), bytes_(0), raw_bytes_(0), source_(source) {}
  ~temp_storage() {
    if (!raw_) return;
    if (source_.acquire) {
      (void)thrust_amd_stream_synchronize(stream_);
      source_.release(source_.ctx, raw_, raw_bytes_);
    } else {
      (void)thrust_amd_temp_release(raw_, stream_);
    }
  }
  void ensure(std::size_t bytes) {
    bytes_ = bytes;
    if (source_.acquire) {
      raw_bytes_ = (bytes ? bytes : 1) + 256;
      raw_ = source_.acquire(source_.ctx, raw_bytes_);
      if (!raw_) throw thrust::system::detail::bad_alloc("the policy's allocator returned a null pointer");
      ptr_ = reinterpret_cast<void*>((reinterpret_cast<std::uintptr_t>(raw_) + 255) / 256 * 256);
      return;
    }
    const int rc = thrust_amd_temp_acquire(&raw_, bytes ? bytes : 1, stream_);
    if (rc != 0) throw thrust::system::detail::bad_alloc(thrust_amd_error_string(rc));
    ptr_ = raw_;
  }
  void* ptr() const { return ptr_; }
  std::size_t* bytes() { return &bytes_; }

 private:
  temp_storage(const temp_storage&);
  temp_storage& operator=(const temp_storage&);
  void* ptr_;
  void* raw_;
  void* stream_;
  std::size_t bytes_, raw_bytes_;
  temp_source source_;
};

// Size query, allocation from the arena with `extra` more bytes at the end (for device
// scalars such as counts), then the run.  call(temp, &bytes) -> status.  Returns the
// address of the extra region.
template <typename Call>
inline void* run(temp_storage& temp, std::size_t extra, const char* what, Call call) {
  std::size_t need = 0;
  throw_on_error(call((void*)nullptr, &need), what);
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + extra);
  *temp.bytes() = aligned;
  throw_on_error(call(temp.ptr(), temp.bytes()), what);
  return static_cast<char*>(temp.ptr()) + aligned;
}

// Mixed element types: the reference converts every element to the accumulator's type as
// it is read and the result to the output's type as it is written.  Here the conversion is
// a pass of its own into (out of) temporary storage; same types cost nothing.
template <typename T, typename V>
inline const T* input_as(const V* in, uint64_t, void*, temp_storage&, std::true_type) {
  return in;
}
template <typename T, typename V>
inline const T* input_as(const V* in, uint64_t n, void* stream, temp_storage& holder, std::false_type) {
  static_assert(is_abi_type<T>::value && is_abi_type<V>::value, "mixed element types must both be arithmetic");
  holder.ensure((std::size_t)n * sizeof(T));
  throw_on_error(thrust_amd_convert(in, dtype_of<V>::value, holder.ptr(), dtype_of<T>::value, n, stream),
                 "element type conversion failed");
  return static_cast<const T*>(holder.ptr());
}
template <typename T, typename V>
inline const T* input_as(const V* in, uint64_t n, void* stream, temp_storage& holder) {
  return input_as<T>(in, n, stream, holder, std::is_same<T, V>());
}
// Where an algorithm that computes in T writes when the caller's output holds U.
template <typename T, typename U>
inline T* output_as(U* out, uint64_t, temp_storage&, std::true_type) {
  return out;
}
template <typename T, typename U>
inline T* output_as(U*, uint64_t n, temp_storage& holder, std::false_type) {
  static_assert(is_abi_type<T>::value && is_abi_type<U>::value, "mixed element types must both be arithmetic");
  holder.ensure((std::size_t)n * sizeof(T));
  return static_cast<T*>(holder.ptr());
}
template <typename T, typename U>
inline T* output_as(U* out, uint64_t n, temp_storage& holder) {
  return output_as<T>(out, n, holder, std::is_same<T, U>());
}
template <typename T, typename U>
inline void finish_output(const T*, U*, uint64_t, void*, std::true_type) {}
template <typename T, typename U>
inline void finish_output(const T* computed, U* out, uint64_t n, void* stream, std::false_type) {
  throw_on_error(thrust_amd_convert(computed, dtype_of<T>::value, out, dtype_of<U>::value, n, stream),
                 "element type conversion failed");
}
template <typename T, typename U>
inline void finish_output(const T* computed, U* out, uint64_t n, void* stream) {
  finish_output(computed, out, n, stream, std::is_same<T, U>());
}

inline void synchronize(void* stream, const char* what) {
  throw_on_error(thrust_amd_stream_synchronize(stream), what);
}

template <typename T>
inline T read_scalar(const void* device_src, void* stream, const char* what) {
  T v;
  throw_on_error(thrust_amd_memcpy(&v, device_src, sizeof(T), THRUST_AMD_D2H, stream), what);
  return v;
}

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
