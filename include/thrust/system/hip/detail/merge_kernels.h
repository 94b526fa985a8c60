// Merge-path merge of two sorted ranges (merge, merge_by_key) as a template on the comparator.
// libthrust_amd.so instantiates it for operator< / operator> behind thrust_amd_merge and
// thrust_amd_merge_by_key; a translation unit compiled with hipcc instantiates it for its own
// comparator and key type.
//
//   partition  one thread per output-tile boundary d = tile * TILE binary-searches the
//              merge path: how many of the first d outputs come from range A
//   merge      a workgroup stages the two sub-ranges of its tile in LDS, every lane finds
//              its own start on the path by binary search in LDS and merges ITEMS
//              elements serially; values follow through LDS by the recorded source slot
//
// Tie rule: an element of B is taken only when comp(b, a) holds, so equal elements of A
// come first (thrust/system/detail/sequential/merge.inl:56-65; the reference's GPU
// serial_merge does the same, thrust/system/cuda/detail/merge.h:111-116).
//
// HBM traffic: (na + nb) * (key + value) read and the same written, plus 8 bytes per tile.
// Replaces the PartitionAgent / MergeAgent pair of thrust/system/cuda/detail/merge.h:152-660.
#pragma once
#include "device_primitives.h"

namespace thrust {
namespace system {
namespace hip {
namespace merging {
using namespace ::thrust::system::hip::prim;

constexpr int MERGE_BLOCK = 256;
constexpr int MERGE_ITEMS = 16;
constexpr int MERGE_TILE = MERGE_BLOCK * MERGE_ITEMS;

// Number of elements taken from A among the first `diag` outputs.
template <typename T, typename PA, typename PB, typename Comp>
THRUST_AMD_DEVICE uint64_t merge_path(PA a, uint64_t na, PB b, uint64_t nb, uint64_t diag, Comp& comp) {
  uint64_t lo = diag > nb ? diag - nb : 0;
  uint64_t hi = diag < na ? diag : na;
  while (lo < hi) {
    const uint64_t mid = (lo + hi) >> 1;
    const T ka = a[mid];
    const T kb = b[diag - 1 - mid];
    if (!comp(kb, ka)) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

template <typename T, typename Comp>
__global__ __launch_bounds__(256) void merge_partition_kernel(const T* __restrict__ a, uint64_t na,
                                                              const T* __restrict__ b, uint64_t nb,
                                                              uint64_t tiles, Comp comp,
                                                              uint64_t* __restrict__ a_split) {
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t > tiles) return;
  const uint64_t total = na + nb;
  uint64_t diag = t * MERGE_TILE;
  if (diag > total) diag = total;
  // the merge-path search of merge_path() below, over the whole ranges: probes shared between threads
  a_split[t] = aligned_partition_point(diag > nb ? diag - nb : 0, diag < na ? diag : na, [&](uint64_t mid) {
    const T ka = a[mid];
    const T kb = b[diag - 1 - mid];
    return !comp(kb, ka);
  });
}

// Slot of output element e in the LDS exchange buffer: one spare slot after every
// MERGE_ITEMS keeps both access patterns off the same banks (lane t writes its run
// t*ITEMS .. t*ITEMS+ITEMS-1, i.e. slots t*(ITEMS+1)+o; the write-out reads consecutive e).
THRUST_AMD_DEVICE uint32_t merge_slot(uint32_t e) { return e + e / MERGE_ITEMS; }
constexpr int MERGE_SLOTS = MERGE_TILE + MERGE_TILE / MERGE_ITEMS + 1;

template <typename T, typename V, bool HAS_VALUES, typename Comp>
__global__ __launch_bounds__(MERGE_BLOCK) void merge_kernel(
    const T* __restrict__ a, uint64_t na, const T* __restrict__ b, uint64_t nb,
    const V* __restrict__ va, const V* __restrict__ vb, T* __restrict__ out, V* __restrict__ vout,
    Comp comp, const uint64_t* __restrict__ a_split) {
  constexpr size_t ITEM = (HAS_VALUES && sizeof(V) > sizeof(T)) ? sizeof(V) : sizeof(T);
  __shared__ __attribute__((aligned(16))) unsigned char s_raw[(size_t)MERGE_SLOTS * ITEM];
  T* s_keys = reinterpret_cast<T*>(s_raw);
  V* s_vals = reinterpret_cast<V*>(s_raw);

  const uint64_t tile = blockIdx.x;
  const uint64_t total = na + nb;
  const uint64_t d0 = tile * MERGE_TILE;
  const uint64_t d1 = (d0 + MERGE_TILE < total) ? d0 + MERGE_TILE : total;
  const uint64_t a0 = a_split[tile], a1 = a_split[tile + 1];
  const uint64_t b0 = d0 - a0, b1 = d1 - a1;
  const uint32_t ca = (uint32_t)(a1 - a0), cb = (uint32_t)(b1 - b0);
  const uint32_t count = ca + cb;  // == d1 - d0

  // ---- stage the keys: A's part first, then B's
  {
    T in[MERGE_ITEMS];
#pragma unroll
    for (int q = 0; q < MERGE_ITEMS; ++q) {
      const uint32_t e = q * MERGE_BLOCK + threadIdx.x;
      in[q] = (e < ca) ? a[a0 + e] : (e < count) ? b[b0 + (e - ca)] : T{};
    }
#pragma unroll
    for (int q = 0; q < MERGE_ITEMS; ++q) s_keys[q * MERGE_BLOCK + threadIdx.x] = in[q];
  }
  __syncthreads();

  // ---- this lane's start on the path, then a serial merge of ITEMS elements
  const uint32_t run0 = threadIdx.x * MERGE_ITEMS;
  const uint32_t diag = run0 < count ? run0 : count;
  uint32_t i = (uint32_t)merge_path<T>(s_keys, (uint64_t)ca, s_keys + ca, (uint64_t)cb, (uint64_t)diag, comp);
  uint32_t j = ca + (diag - i);  // slot of the next element of B's part
  T k[MERGE_ITEMS];
  uint32_t src[MERGE_ITEMS];
  // slots past the parts hold staged padding (or the one slack slot): reads stay in bounds
  T ka = s_keys[i];
  T kb = s_keys[j];
#pragma unroll
  for (int o = 0; o < MERGE_ITEMS; ++o) {
    const bool take_b = (j < count) && (i >= ca || comp(kb, ka));
    k[o] = take_b ? kb : ka;
    src[o] = take_b ? j : i;
    const uint32_t next = take_b ? ++j : ++i;
    const T nk = s_keys[next];  // next <= count <= MERGE_TILE
    if (take_b) kb = nk;
    else ka = nk;
  }
  __syncthreads();  // all keys have been read from the staging area

  // ---- keys leave through LDS so that consecutive lanes write consecutive addresses
#pragma unroll
  for (int o = 0; o < MERGE_ITEMS; ++o) s_keys[merge_slot(run0 + o)] = k[o];
  __syncthreads();
#pragma unroll
  for (int q = 0; q < MERGE_ITEMS; ++q) {
    const uint32_t e = q * MERGE_BLOCK + threadIdx.x;
    if (e < count) out[d0 + e] = s_keys[merge_slot(e)];
  }

  if constexpr (HAS_VALUES) {
    __syncthreads();  // key write-out has read the exchange buffer
    {
      V in[MERGE_ITEMS];
#pragma unroll
      for (int q = 0; q < MERGE_ITEMS; ++q) {
        const uint32_t e = q * MERGE_BLOCK + threadIdx.x;
        in[q] = (e < ca) ? va[a0 + e] : (e < count) ? vb[b0 + (e - ca)] : V{};
      }
#pragma unroll
      for (int q = 0; q < MERGE_ITEMS; ++q) s_vals[q * MERGE_BLOCK + threadIdx.x] = in[q];
    }
    __syncthreads();
    V v[MERGE_ITEMS];
#pragma unroll
    for (int o = 0; o < MERGE_ITEMS; ++o) v[o] = s_vals[src[o]];  // src[o] < count for valid outputs
    __syncthreads();
#pragma unroll
    for (int o = 0; o < MERGE_ITEMS; ++o) s_vals[merge_slot(run0 + o)] = v[o];
    __syncthreads();
#pragma unroll
    for (int q = 0; q < MERGE_ITEMS; ++q) {
      const uint32_t e = q * MERGE_BLOCK + threadIdx.x;
      if (e < count) vout[d0 + e] = s_vals[merge_slot(e)];
    }
  }
}

// Bytes of temporary storage for merging `total` elements: the tile boundaries on the merge path.
inline size_t merge_temp_bytes(uint64_t total) {
  const uint64_t tiles = (total + MERGE_TILE - 1) / MERGE_TILE;
  return align_up((size_t)(tiles + 1) * sizeof(uint64_t), 256);
}

// Both kernels.  `split` holds merge_temp_bytes(na + nb) bytes; total > 0.
template <typename T, typename V, bool HAS_VALUES, typename Comp>
inline int merge_launch(uint64_t* split, const T* a, uint64_t na, const T* b, uint64_t nb, const V* va, const V* vb,
                        T* out, V* vout, Comp comp, hipStream_t stream) {
  const uint64_t total = na + nb;
  const uint64_t tiles = (total + MERGE_TILE - 1) / MERGE_TILE;
  if (tiles > 0x7fffffffull) return (int)hipErrorInvalidValue;
  THRUST_AMD_KERNEL_LAUNCH("merge_partition", stream, (merge_partition_kernel<T, Comp>),
                           dim3((uint32_t)((tiles + 1 + 255) / 256)), dim3(256), a, na, b, nb, tiles, comp, split);
  hipError_t e = hipPeekAtLastError();
  if (e != hipSuccess) return (int)e;
  THRUST_AMD_KERNEL_LAUNCH("merge", stream, (merge_kernel<T, V, HAS_VALUES, Comp>), dim3((uint32_t)tiles),
                           dim3(MERGE_BLOCK), a, na, b, nb, va, vb, out, vout, comp, (const uint64_t*)split);
  return (int)hipPeekAtLastError();
}

}  // namespace merging
}  // namespace hip
}  // namespace system
}  // namespace thrust
