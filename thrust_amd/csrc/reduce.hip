// thrust_amd_reduce: two-kernel tree reduction.
//
//   kernel 1  grid-stride over tiles of BLOCK*VEC*UNROLL elements; every lane issues
//             UNROLL independent 16-byte loads per tile, folds them into one register
//             accumulator, then wave64 DPP reduction -> LDS across the waves -> one
//             partial per workgroup.
//   kernel 2  one workgroup folds init and the partials and writes *d_out.
//
// HBM traffic: n*sizeof(T) read, (grid+1)*sizeof(T) written -- the kernel is bound by
// the read stream alone.  Replaces the ReduceAgent pair of the reference
// (thrust/system/cuda/detail/reduce.h:151-665) and cub::DispatchReduce (:946-954).
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"
#include "reduce_common.hpp"

namespace ta {

template <typename T, typename Op, bool ALIGNED>
__global__ __launch_bounds__(REDUCE_BLOCK) void reduce_partials_kernel(const T* __restrict__ in,
                                                                       uint64_t n,
                                                                       T* __restrict__ partials) {
  constexpr int VEC = Vec16<T>::N;
  constexpr uint64_t TILE = (uint64_t)REDUCE_BLOCK * VEC * REDUCE_UNROLL;
  const Op op;
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
      for (int i = 0; i < VEC; ++i) acc = op(acc, x[u].v[i]);
    }
  }
  // Ragged tail (< TILE elements): element-wise, spread over the first workgroups.
  const uint64_t tail_begin = full_tiles * TILE;
  for (uint64_t i = tail_begin + (uint64_t)blockIdx.x * REDUCE_BLOCK + threadIdx.x; i < n;
       i += (uint64_t)gridDim.x * REDUCE_BLOCK)
    acc = op(acc, in[i]);

  __shared__ T lds[REDUCE_BLOCK / WAVE];
  const T r = block_reduce<REDUCE_BLOCK>(acc, op, lds);
  if (threadIdx.x == 0) partials[blockIdx.x] = r;
}

struct ReduceLaunch {
  template <typename T, typename Op>
  static int run(void* temp, const void* in, uint64_t n, const void* init, void* d_out,
                 hipStream_t stream) {
    T init_v;
    __builtin_memcpy(&init_v, init, sizeof(T));
    T* partials = static_cast<T*>(temp);
    const uint32_t grid = reduce_grid(n, sizeof(T));
    const T* src = static_cast<const T*>(in);
    if (n == 0) {
      TA_LAUNCH("reduce_final", stream, (reduce_final_kernel<T, Op>), dim3(1), dim3(REDUCE_BLOCK), partials, 0u, init_v, static_cast<T*>(d_out));
      TA_CHECK_LAUNCH();
      return 0;
    }
    if (is_aligned16(in))
      TA_LAUNCH("reduce_partials", stream, (reduce_partials_kernel<T, Op, true>), dim3(grid), dim3(REDUCE_BLOCK), src, n, partials);
    else
      TA_LAUNCH("reduce_partials", stream, (reduce_partials_kernel<T, Op, false>), dim3(grid), dim3(REDUCE_BLOCK), src, n, partials);
    TA_CHECK_LAUNCH();
    TA_LAUNCH("reduce_final", stream, (reduce_final_kernel<T, Op>), dim3(1), dim3(REDUCE_BLOCK), partials, grid, init_v, static_cast<T*>(d_out));
    TA_CHECK_LAUNCH();
    return 0;
  }
};

}  // namespace ta

TA_EXPORT int thrust_amd_reduce(void* temp, size_t* temp_bytes, const void* in, uint64_t n,
                                 int dtype, int op, const void* init, void* d_out, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(dtype) || !valid_binop(op)) return (int)hipErrorInvalidValue;
  const size_t elem = thrust_amd_dtype_size(dtype);
  const size_t need = align_up((size_t)NUM_CU * REDUCE_BLOCKS_PER_CU * elem, 256);
  if (temp == nullptr) {
    *temp_bytes = need;
    return 0;
  }
  if (*temp_bytes < need || !init || !d_out || (n && !in)) return (int)hipErrorInvalidValue;
  return dispatch_dtype_op<ReduceLaunch>(dtype, op, temp, in, n, init, d_out, (hipStream_t)stream);
}
