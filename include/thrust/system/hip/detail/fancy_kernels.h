// Element-wise kernels that take iterators and functors by value: materialisation of a
// fancy iterator, for_each, binary transform, scatter.  They are templates on types only
// the user's translation unit knows, so they exist where that unit is compiled with hipcc
// (the reference instantiates its kernels the same way: thrust/system/cuda/detail/core/
// util.h:527-561 LoadIterator, parallel_for.h).  HBM traffic: what the iterators read and
// one write per element.
#pragma once
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

inline int launch_status() { return (int)hipPeekAtLastError(); }

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
