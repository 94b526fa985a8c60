// Pieces shared by the reduction kernels: workgroup fold, the final one-workgroup kernel
// and the grid size (a few workgroups per CU, each folding many tiles).
#pragma once
#include "common.hpp"

namespace ta {

constexpr int REDUCE_BLOCK = 256;
constexpr int REDUCE_UNROLL = 8;
constexpr int REDUCE_BLOCKS_PER_CU = 8;

// Folds the values of a whole workgroup; result valid in thread 0.
template <int BLOCK, typename T, typename Op>
TA_DEVICE T block_reduce(T v, Op op, T* lds /* BLOCK/64 slots */) {
  constexpr int WAVES = BLOCK / WAVE;
  v = wave_reduce(v, op);
  const int wave = threadIdx.x / WAVE;
  if ((threadIdx.x % WAVE) == 0) lds[wave] = v;
  __syncthreads();
  T r = lds[0];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) r = op(r, lds[w]);
  return r;
}

template <typename T, typename Op>
__global__ __launch_bounds__(REDUCE_BLOCK) void reduce_final_kernel(const T* __restrict__ partials,
                                                                    uint32_t count, T init,
                                                                    T* __restrict__ out) {
  const Op op;
  T acc = Op::template identity<T>();
  for (uint32_t i = threadIdx.x; i < count; i += REDUCE_BLOCK) acc = op(acc, partials[i]);
  __shared__ T lds[REDUCE_BLOCK / WAVE];
  const T r = block_reduce<REDUCE_BLOCK>(acc, op, lds);
  if (threadIdx.x == 0) *out = op(init, r);
}

static inline uint32_t reduce_grid(uint64_t n, size_t elem) {
  const uint64_t tile = (uint64_t)REDUCE_BLOCK * (16 / elem) * REDUCE_UNROLL;
  uint64_t tiles = (n + tile - 1) / tile;
  const uint64_t cap = (uint64_t)NUM_CU * REDUCE_BLOCKS_PER_CU;
  if (tiles < 1) tiles = 1;
  return (uint32_t)(tiles < cap ? tiles : cap);
}

}  // namespace ta
