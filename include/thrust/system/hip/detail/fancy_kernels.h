// Element-wise kernels that take iterators and functors by value: materialisation of a
// fancy iterator, for_each, binary transform, scatter.  They are templates on types only
// the user's translation unit knows, so they exist where that unit is compiled with hipcc
// (the reference instantiates its kernels the same way: thrust/system/cuda/detail/core/
// util.h:527-561 LoadIterator, parallel_for.h).  HBM traffic: what the iterators read and
// one write per element.
#pragma once
#include <type_traits>
#if !defined(__HIPCC__)
#error "thrust/system/hip/detail/fancy_kernels.h is HIP code: compile this translation unit with hipcc"
#endif
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace thrust {
namespace system {
namespace hip {
namespace detail {

constexpr int ELEMENTWISE_BLOCK = 256;
inline unsigned elementwise_grid(uint64_t n) {
  const uint64_t blocks = (n + ELEMENTWISE_BLOCK - 1) / ELEMENTWISE_BLOCK;
  const uint64_t cap = (uint64_t)1 << 20;  // one element per lane up to 2^28 (many short workgroups keep more
                                           // memory requests in flight than a few that loop); grid-stride beyond
  return (unsigned)(blocks < 1 ? 1 : (blocks < cap ? blocks : cap));
}

// out may be a pointer or a zip of pointers: out[i] is then a tuple of references, written through
template <typename View, typename OutView>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void materialize_kernel(View first, OutView out, uint64_t n) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = first[i];
}

template <typename View, typename F>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void for_each_kernel(View first, uint64_t n, F f) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) f(first[i]);
}

// (the functor receives the element itself, so a functor that modifies its argument -- `++_1`
// -- changes the input, as it does in the reference)
template <typename View, typename OutView, typename F>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void transform1_kernel(View in, OutView out, uint64_t n, F f) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = f(in[i]);
}

template <typename ViewA, typename ViewB, typename OutView, typename F>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void transform2_kernel(ViewA a, ViewB b, OutView out, uint64_t n, F f) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = f(a[i], b[i]);
}

template <typename ViewIn, typename ViewMap, typename OutView>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void scatter_kernel(ViewIn in, ViewMap map, OutView out, uint64_t n) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[map[i]] = in[i];
}

// ---- arrays of 4- and 8-byte elements: every thread takes PER consecutive elements, 16 bytes at a
// time.  The functor receives the element where it lies in memory, exactly as in the plain kernels
// above (it may take its address, or change it: thrust/system/cuda/detail/for_each.h:58 hands it
// raw_reference_cast(input[idx])); the element accesses of one thread are adjacent and 16-byte
// aligned, which is what lets the compiler fetch them with one load.  Results leave as one 16-byte
// store after the thread's PER calls, so an output that is the input ends up holding the results,
// as in `*result = f(*first)`.
template <typename T, int N>
struct alignas(sizeof(T) * N >= 16 ? 16 : sizeof(T) * N) element_pack {
  T v[N];
};
template <typename T>
struct is_packable : std::integral_constant<bool, std::is_trivially_copyable<T>::value && (sizeof(T) == 4 || sizeof(T) == 8)> {};
template <typename T, int PER>
__device__ __forceinline__ T* pack_at(T* base, uint64_t p) {
  constexpr size_t BYTES = sizeof(T) * PER >= 16 ? 16 : sizeof(T) * PER;
  return static_cast<T*>(__builtin_assume_aligned(base, BYTES)) + p * PER;
}

template <typename PA, typename O, typename F, int PER>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void transform1_packed_kernel(PA in, O* out, uint64_t n, F f) {
  const uint64_t packs = n / PER;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; p < packs; p += stride) {
    auto* a = pack_at<typename std::remove_pointer<PA>::type, PER>(in, p);
    element_pack<O, PER> o;
#pragma unroll
    for (int k = 0; k < PER; ++k) o.v[k] = f(a[k]);
    reinterpret_cast<element_pack<O, PER>*>(out)[p] = o;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0)
    for (uint64_t i = packs * PER; i < n; ++i) out[i] = f(in[i]);
}
template <typename PA, typename PB, typename O, typename F, int PER>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void transform2_packed_kernel(PA ina, PB inb, O* out, uint64_t n, F f) {
  const uint64_t packs = n / PER;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; p < packs; p += stride) {
    auto* a = pack_at<typename std::remove_pointer<PA>::type, PER>(ina, p);
    auto* b = pack_at<typename std::remove_pointer<PB>::type, PER>(inb, p);
    element_pack<O, PER> o;
#pragma unroll
    for (int k = 0; k < PER; ++k) o.v[k] = f(a[k], b[k]);
    reinterpret_cast<element_pack<O, PER>*>(out)[p] = o;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0)
    for (uint64_t i = packs * PER; i < n; ++i) out[i] = f(ina[i], inb[i]);
}
template <typename PA, typename F, int PER>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void for_each_packed_kernel(PA first, uint64_t n, F f) {
  const uint64_t packs = n / PER;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; p < packs; p += stride) {
    auto* a = pack_at<typename std::remove_pointer<PA>::type, PER>(first, p);
#pragma unroll
    for (int k = 0; k < PER; ++k) f(a[k]);
  }
  if (blockIdx.x == 0 && threadIdx.x == 0)
    for (uint64_t i = packs * PER; i < n; ++i) f(first[i]);
}

// out[0] = in[0], out[i] = f(in[i], in[i - 1]); `in` and `out` do not overlap
template <typename A, typename O, typename F, int PER>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void adjacent_packed_kernel(const A* in, O* out, uint64_t n, F f) {
  const uint64_t packs = n / PER;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; p < packs; p += stride) {
    const element_pack<A, PER> a = reinterpret_cast<const element_pack<A, PER>*>(in)[p];
    element_pack<O, PER> o;
    if (p == 0) o.v[0] = a.v[0];
    else o.v[0] = f(a.v[0], in[p * PER - 1]);
#pragma unroll
    for (int k = 1; k < PER; ++k) o.v[k] = f(a.v[k], a.v[k - 1]);
    reinterpret_cast<element_pack<O, PER>*>(out)[p] = o;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0)
    for (uint64_t i = packs * PER; i < n; ++i) out[i] = i ? (O)f(in[i], in[i - 1]) : (O)in[i];
}

template <typename T>
inline bool pack_aligned(const T* p, int per) {
  const size_t bytes = sizeof(T) * (size_t)per;
  return reinterpret_cast<uintptr_t>(p) % (bytes >= 16 ? 16 : bytes) == 0;
}

inline int launch_status() { return (int)hipPeekAtLastError(); }

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
