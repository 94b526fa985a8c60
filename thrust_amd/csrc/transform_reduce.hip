// thrust_amd_transform_reduce / thrust_amd_count_if / thrust_amd_inner_product: reductions
// of a value computed on the fly from one or two input streams, with the two-kernel tree
// of thrust_amd_reduce.
//
//   transform_reduce  init OP f(x[0]) OP ... with f one of identity / negate / square
//   count_if          number of elements with (x CMP threshold), as a 64-bit count
//   inner_product     init + sum of a[i] * b[i], products and sums in the element type
//                     (integers wrap modulo 2^bits)
//
// The reference builds the other two on transform_reduce (reduce over a transform
// iterator, thrust/system/detail/generic/transform_reduce.inl:30-48): count_if maps each
// element to 0/1 of the difference type and adds (thrust/system/detail/generic/count.inl:45-67),
// and inner_product multiplies with multiplies<T> and adds with plus<T>, T being the type of
// init (thrust/system/detail/generic/inner_product.inl:33-72); on the device all three end in
// reduce_n (thrust/system/cuda/detail/transform_reduce.h, inner_product.h).
//
// HBM traffic: every input element is read once; a few KB of partials are written.
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"
#include "reduce_common.hpp"

namespace ta {

// The comparison is a template parameter: one kernel per (type, comparison), so that the
// inner loop is a single compare and add.
template <int CMP, typename T>
TA_DEVICE bool compare_fixed(T x, T t) {
  if constexpr (CMP == THRUST_AMD_LT) return x < t;
  else if constexpr (CMP == THRUST_AMD_LE) return x <= t;
  else if constexpr (CMP == THRUST_AMD_GT) return x > t;
  else if constexpr (CMP == THRUST_AMD_GE) return x >= t;
  else if constexpr (CMP == THRUST_AMD_EQ) return x == t;
  else if constexpr (CMP == THRUST_AMD_NE) return x != t;
  else return x != (T)0;
}

template <typename T, int CMP, bool ALIGNED>
__global__ __launch_bounds__(REDUCE_BLOCK) void count_if_partials_kernel(const T* __restrict__ in,
                                                                         uint64_t n, T threshold,
                                                                         uint64_t* __restrict__ partials) {
  constexpr int VEC = Vec16<T>::N;
  constexpr uint64_t TILE = (uint64_t)REDUCE_BLOCK * VEC * REDUCE_UNROLL;
  uint64_t acc = 0;
  const uint64_t full_tiles = n / TILE;
  for (uint64_t tile = blockIdx.x; tile < full_tiles; tile += gridDim.x) {
    const T* base = in + tile * TILE + (uint64_t)threadIdx.x * VEC;
    Vec16<T> x[REDUCE_UNROLL];
#pragma unroll
    for (int u = 0; u < REDUCE_UNROLL; ++u)
      x[u] = load_vec<ALIGNED>(base + (uint64_t)u * REDUCE_BLOCK * VEC);
    uint32_t c = 0;  // at most VEC * UNROLL per tile
#pragma unroll
    for (int u = 0; u < REDUCE_UNROLL; ++u) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) c += compare_fixed<CMP>(x[u].v[i], threshold) ? 1u : 0u;
    }
    acc += c;
  }
  const uint64_t tail_begin = full_tiles * TILE;
  for (uint64_t i = tail_begin + (uint64_t)blockIdx.x * REDUCE_BLOCK + threadIdx.x; i < n;
       i += (uint64_t)gridDim.x * REDUCE_BLOCK)
    acc += compare_fixed<CMP>(in[i], threshold) ? 1u : 0u;

  __shared__ uint64_t lds[REDUCE_BLOCK / WAVE];
  const uint64_t r = block_reduce<REDUCE_BLOCK>(acc, OpPlus{}, lds);
  if (threadIdx.x == 0) partials[blockIdx.x] = r;
}

// reduce_partials_kernel of thrust_amd_reduce with `un` applied to every element first.
template <typename T, typename Un, typename Op, bool ALIGNED>
__global__ __launch_bounds__(REDUCE_BLOCK) void transform_reduce_partials_kernel(const T* __restrict__ in,
                                                                                 uint64_t n,
                                                                                 T* __restrict__ partials) {
  constexpr int VEC = Vec16<T>::N;
  constexpr uint64_t TILE = (uint64_t)REDUCE_BLOCK * VEC * REDUCE_UNROLL;
  const Op op;
  const Un un;
  T acc = Op::template identity<T>();
  const uint64_t full_tiles = n / TILE;
  for (uint64_t tile = blockIdx.x; tile < full_tiles; tile += gridDim.x) {
    const T* base = in + tile * TILE + (uint64_t)threadIdx.x * VEC;
    Vec16<T> x[REDUCE_UNROLL];
#pragma unroll
    for (int u = 0; u < REDUCE_UNROLL; ++u)
      x[u] = load_vec<ALIGNED>(base + (uint64_t)u * REDUCE_BLOCK * VEC);
#pragma unroll
    for (int u = 0; u < REDUCE_UNROLL; ++u) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc = op(acc, un(x[u].v[i]));
    }
  }
  const uint64_t tail_begin = full_tiles * TILE;
  for (uint64_t i = tail_begin + (uint64_t)blockIdx.x * REDUCE_BLOCK + threadIdx.x; i < n;
       i += (uint64_t)gridDim.x * REDUCE_BLOCK)
    acc = op(acc, un(in[i]));

  __shared__ T lds[REDUCE_BLOCK / WAVE];
  const T r = block_reduce<REDUCE_BLOCK>(acc, op, lds);
  if (threadIdx.x == 0) partials[blockIdx.x] = r;
}

template <typename T, bool ALIGNED>
__global__ __launch_bounds__(REDUCE_BLOCK) void inner_product_partials_kernel(const T* __restrict__ a,
                                                                              const T* __restrict__ b,
                                                                              uint64_t n,
                                                                              T* __restrict__ partials) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int UNROLL = REDUCE_UNROLL / 2;  // two streams: the same number of loads in flight
  constexpr uint64_t TILE = (uint64_t)REDUCE_BLOCK * VEC * UNROLL;
  const OpPlus op;
  T acc = OpPlus::identity<T>();
  const uint64_t full_tiles = n / TILE;
  for (uint64_t tile = blockIdx.x; tile < full_tiles; tile += gridDim.x) {
    const uint64_t off = tile * TILE + (uint64_t)threadIdx.x * VEC;
    Vec16<T> x[UNROLL], y[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      x[u] = load_vec<ALIGNED>(a + off + (uint64_t)u * REDUCE_BLOCK * VEC);
      y[u] = load_vec<ALIGNED>(b + off + (uint64_t)u * REDUCE_BLOCK * VEC);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc = op(acc, mul_wrap(x[u].v[i], y[u].v[i]));
    }
  }
  const uint64_t tail_begin = full_tiles * TILE;
  for (uint64_t i = tail_begin + (uint64_t)blockIdx.x * REDUCE_BLOCK + threadIdx.x; i < n;
       i += (uint64_t)gridDim.x * REDUCE_BLOCK)
    acc = op(acc, mul_wrap(a[i], b[i]));

  __shared__ T lds[REDUCE_BLOCK / WAVE];
  const T r = block_reduce<REDUCE_BLOCK>(acc, op, lds);
  if (threadIdx.x == 0) partials[blockIdx.x] = r;
}

static size_t transform_reduce_temp(size_t elem) {
  return align_up((size_t)NUM_CU * REDUCE_BLOCKS_PER_CU * elem, 256);
}

}  // namespace ta

TA_EXPORT int thrust_amd_transform_reduce(void* temp, size_t* temp_bytes, const void* in, uint64_t n,
                                          int dtype, int unary, int op, const void* init,
                                          void* d_out, void* stream_v) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(dtype) || !valid_unary(unary) || !valid_binop(op))
    return (int)hipErrorInvalidValue;
  if (unary == THRUST_AMD_IDENTITY)
    return thrust_amd_reduce(temp, temp_bytes, in, n, dtype, op, init, d_out, stream_v);
  const size_t need = transform_reduce_temp(thrust_amd_dtype_size(dtype));
  if (temp == nullptr) {
    *temp_bytes = need;
    return 0;
  }
  if (*temp_bytes < need || !init || !d_out || (n && !in)) return (int)hipErrorInvalidValue;
  hipStream_t stream = (hipStream_t)stream_v;
  return with_dtype(dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_transform(unary, [&](auto un) {
      using Un = decltype(un);
      return with_binop(op, [&](auto o) {
        using Op = decltype(o);
        T init_v;
        __builtin_memcpy(&init_v, init, sizeof(T));
        T* partials = static_cast<T*>(temp);
        uint32_t grid = 0;
        if (n) {
          grid = reduce_grid(n, sizeof(T));
          const T* src = static_cast<const T*>(in);
          if (is_aligned16(in))
            TA_LAUNCH("transform_reduce_partials", stream, (transform_reduce_partials_kernel<T, Un, Op, true>), dim3(grid), dim3(REDUCE_BLOCK), src, n, partials);
          else
            TA_LAUNCH("transform_reduce_partials", stream, (transform_reduce_partials_kernel<T, Un, Op, false>), dim3(grid), dim3(REDUCE_BLOCK), src, n, partials);
          TA_CHECK_LAUNCH();
        }
        TA_LAUNCH("reduce_final", stream, (reduce_final_kernel<T, Op>), dim3(1), dim3(REDUCE_BLOCK), (const T*)partials, grid, init_v, static_cast<T*>(d_out));
        TA_CHECK_LAUNCH();
        return 0;
      });
    });
  });
}

TA_EXPORT int thrust_amd_count_if(void* temp, size_t* temp_bytes, const void* in, uint64_t n, int dtype,
                                  int cmp, const void* threshold, uint64_t* d_count, void* stream_v) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(dtype) || !valid_cmp(cmp)) return (int)hipErrorInvalidValue;
  const size_t need = transform_reduce_temp(sizeof(uint64_t));
  if (temp == nullptr) {
    *temp_bytes = need;
    return 0;
  }
  if (*temp_bytes < need || !d_count || (n && !in) || (cmp != THRUST_AMD_NONZERO && !threshold))
    return (int)hipErrorInvalidValue;
  hipStream_t stream = (hipStream_t)stream_v;
  return with_dtype(dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    T thr{};
    if (threshold) __builtin_memcpy(&thr, threshold, sizeof(T));
    uint64_t* partials = static_cast<uint64_t*>(temp);
    uint32_t grid = 0;
    if (n) {
      grid = reduce_grid(n, sizeof(T));
      const T* src = static_cast<const T*>(in);
      auto launch = [&](auto cmp_tag) {
        constexpr int CMP = decltype(cmp_tag)::value;
        if (is_aligned16(in))
          TA_LAUNCH("count_if_partials", stream, (count_if_partials_kernel<T, CMP, true>), dim3(grid), dim3(REDUCE_BLOCK), src, n, thr, partials);
        else
          TA_LAUNCH("count_if_partials", stream, (count_if_partials_kernel<T, CMP, false>), dim3(grid), dim3(REDUCE_BLOCK), src, n, thr, partials);
      };
      switch (cmp) {
        case THRUST_AMD_LT: launch(std::integral_constant<int, THRUST_AMD_LT>{}); break;
        case THRUST_AMD_LE: launch(std::integral_constant<int, THRUST_AMD_LE>{}); break;
        case THRUST_AMD_GT: launch(std::integral_constant<int, THRUST_AMD_GT>{}); break;
        case THRUST_AMD_GE: launch(std::integral_constant<int, THRUST_AMD_GE>{}); break;
        case THRUST_AMD_EQ: launch(std::integral_constant<int, THRUST_AMD_EQ>{}); break;
        case THRUST_AMD_NE: launch(std::integral_constant<int, THRUST_AMD_NE>{}); break;
        default: launch(std::integral_constant<int, THRUST_AMD_NONZERO>{}); break;
      }
      TA_CHECK_LAUNCH();
    }
    TA_LAUNCH("reduce_final", stream, (reduce_final_kernel<uint64_t, OpPlus>), dim3(1), dim3(REDUCE_BLOCK), (const uint64_t*)partials, grid, (uint64_t)0, d_count);
    TA_CHECK_LAUNCH();
    return 0;
  });
}

TA_EXPORT int thrust_amd_inner_product(void* temp, size_t* temp_bytes, const void* a, const void* b,
                                       uint64_t n, int dtype, const void* init, void* d_out,
                                       void* stream_v) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(dtype)) return (int)hipErrorInvalidValue;
  const size_t need = transform_reduce_temp(thrust_amd_dtype_size(dtype));
  if (temp == nullptr) {
    *temp_bytes = need;
    return 0;
  }
  if (*temp_bytes < need || !init || !d_out || (n && (!a || !b))) return (int)hipErrorInvalidValue;
  hipStream_t stream = (hipStream_t)stream_v;
  return with_dtype(dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    T init_v;
    __builtin_memcpy(&init_v, init, sizeof(T));
    T* partials = static_cast<T*>(temp);
    uint32_t grid = 0;
    if (n) {
      grid = reduce_grid(n, sizeof(T));
      const T* pa = static_cast<const T*>(a);
      const T* pb = static_cast<const T*>(b);
      if (is_aligned16(a) && is_aligned16(b))
        TA_LAUNCH("inner_product_partials", stream, (inner_product_partials_kernel<T, true>), dim3(grid), dim3(REDUCE_BLOCK), pa, pb, n, partials);
      else
        TA_LAUNCH("inner_product_partials", stream, (inner_product_partials_kernel<T, false>), dim3(grid), dim3(REDUCE_BLOCK), pa, pb, n, partials);
      TA_CHECK_LAUNCH();
    }
    TA_LAUNCH("reduce_final", stream, (reduce_final_kernel<T, OpPlus>), dim3(1), dim3(REDUCE_BLOCK), (const T*)partials, grid, init_v, static_cast<T*>(d_out));
    TA_CHECK_LAUNCH();
    return 0;
  });
}
