// Single-pass prefix scan with decoupled look-back for a caller's operator (hipcc translation
// units): any associative operator on elements of 4 or 8 bytes.  The operator need not commute
// and need not have an identity: operands are only ever combined in input order, and "nothing
// before this" is a case of its own (decided by lane, wave and tile number, all known without
// looking at data) instead of an identity element.  libthrust_amd.so has its own instantiations
// of this scheme for plus / minimum / maximum, which use the identity and the commutativity
// (thrust_amd_inclusive_scan, thrust_amd_exclusive_scan); this header serves every other operator.
// The reference passes the operator into its scan agent the same way
// (thrust/system/cuda/detail/scan.h:198-640).
//
// Tile order is a dynamic ticket (one atomic per workgroup), so a tile only ever waits for tiles
// that have already started.  Data layout inside a tile: wave w owns a contiguous span of
// 64*CHUNKS 16-byte vectors; its lane l holds vectors l, 64+l, 128+l, ... of that span, so every
// global load/store instruction of a wave covers 1 KiB of consecutive addresses.  The scan runs
// as CHUNKS wave scans (DPP) chained by the running total of the wave's span, one step across
// the waves through LDS, and the look-back across tiles.
//
// HBM traffic: n*sizeof(T) read + n*sizeof(T) written; 8*W bytes of tile descriptor per tile
// (W = 32-bit words of T).
#pragma once
#include "device_primitives.h"

namespace thrust {
namespace system {
namespace hip {
namespace scanning {
using namespace ::thrust::system::hip::prim;

struct ScanShapeLarge { static constexpr int BLOCK = 1024, CHUNKS = 12; };
struct ScanShapeSmall { static constexpr int BLOCK = 256, CHUNKS = 4; };
constexpr uint64_t SCAN_LARGE_MIN_BYTES = (uint64_t)32 << 20;

// (a template only so that every translation unit may hold a copy)
template <int = 0>
__global__ void scan_init_kernel(uint64_t* __restrict__ words, uint64_t count, uint32_t* __restrict__ ticket) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) words[i] = 0;
  if (i == 0) *ticket = 0;
}

// Inclusive scan across the wave in lane order without an identity: a lane that has no
// partner at a step keeps its value.
template <typename T, typename Op>
THRUST_AMD_DEVICE T wave_inclusive_scan_ordered(T v, Op& op, int lane) {
  T t;
  t = dpp_move<DPP_ROW_SHR1>(v, v);
  if ((lane & 15) >= 1) v = op(t, v);
  t = dpp_move<DPP_ROW_SHR2>(v, v);
  if ((lane & 15) >= 2) v = op(t, v);
  t = dpp_move<DPP_ROW_SHR4>(v, v);
  if ((lane & 15) >= 4) v = op(t, v);
  t = dpp_move<DPP_ROW_SHR8>(v, v);
  if ((lane & 15) >= 8) v = op(t, v);
  // lane 15 of row r -> all lanes of row r+1 (rows 1 and 3), then lane 31 -> rows 2 and 3
  t = dpp_move<DPP_ROW_BCAST15, 0xa>(v, v);
  if (lane & 16) v = op(t, v);
  t = dpp_move<DPP_ROW_BCAST31, 0xc>(v, v);
  if (lane >= 32) v = op(t, v);
  return v;
}

// A value that may be absent, for the look-back window (lanes whose descriptor does not count).
template <typename T>
struct Maybe {
  uint32_t has;
  T value;
};
template <typename T, typename Op>
struct MaybeOp {
  Op* op;
  THRUST_AMD_DEVICE Maybe<T> operator()(const Maybe<T>& a, const Maybe<T>& b) const {
    Maybe<T> r;
    r.has = a.has | b.has;
    r.value = (a.has && b.has) ? (T)(*op)(a.value, b.value) : (a.has ? a.value : b.value);
    return r;
  }
};

// The look-back of prim::tile_lookback without an identity: the fold, oldest to newest, of
// everything before `tile` (> 0).  Run by one full wave; the result is valid in all lanes.
template <typename T, typename Op>
THRUST_AMD_DEVICE T tile_lookback_ordered(const uint64_t* status_base, uint32_t tile, Op& op) {
  constexpr int W = TileWords<T>::W;
  constexpr int WIN = 8;
  const int lane = lane_id();
  MaybeOp<T, Op> mop{&op};
  Maybe<T> running{0u, T{}};
  int64_t base = (int64_t)tile - 1;
  for (;;) {
    const int64_t idx = base - 63 + lane;
    T val = T{};
    uint32_t st;
    uint64_t needed;
    bool counts;  // this lane inspects a real descriptor
    for (;;) {
      counts = lane >= WAVE - WIN && idx >= 0;
      if (counts) st = tile_try_load<T>(status_base + (size_t)idx * W, val);
      else st = (idx < 0 && lane >= WAVE - WIN) ? (uint32_t)TS_INCLUSIVE : (uint32_t)TS_PARTIAL;
      const uint64_t invalid = __builtin_amdgcn_ballot_w64(st == TS_INVALID);
      const uint64_t incl = __builtin_amdgcn_ballot_w64(st == TS_INCLUSIVE);
      needed = incl ? (~0ull << (63 - __builtin_clzll(incl))) : ~0ull;
      if ((invalid & needed) == 0) {
        const bool found = incl != 0;
        Maybe<T> contrib{(counts && ((needed >> lane) & 1)) ? 1u : 0u, val};
        const Maybe<T> window = readlane(wave_inclusive_scan_ordered(contrib, mop, lane), 63);
        running = mop(window, running);  // the window is older than what was gathered so far
        if (found) return running.value;  // tile > 0: at least tile 0's descriptor was counted
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    base -= WIN;
  }
}

template <typename T, typename Op, bool EXCLUSIVE, bool ALIGNED, typename Shape>
__global__ __launch_bounds__(Shape::BLOCK) void ordered_scan_kernel(const T* in, T* out, uint64_t n, T init, Op op,
                                                                  uint64_t* __restrict__ status,
                                                                  uint32_t* __restrict__ ticket) {
  constexpr int BLOCK = Shape::BLOCK;
  constexpr int CHUNKS = Shape::CHUNKS;
  constexpr int VEC = Vec16<T>::N;
  constexpr int WAVES = BLOCK / WAVE;
  constexpr uint32_t WAVE_SPAN = WAVE * CHUNKS * VEC;  // elements per wave
  constexpr uint32_t TILE = WAVES * WAVE_SPAN;
  constexpr int W = TileWords<T>::W;

  __shared__ uint32_t s_tile;
  __shared__ __attribute__((aligned(16))) unsigned char s_raw[(WAVES + 1) * sizeof(T)];  // T may be a struct of the caller
  T* s_wave_agg = reinterpret_cast<T*>(s_raw);
  T* s_prefix = s_wave_agg + WAVES;

  if (threadIdx.x == 0) s_tile = atomicAdd(ticket, 1u);
  __syncthreads();
  const uint32_t tile = s_tile;
  const uint64_t tile_base = (uint64_t)tile * TILE;
  const uint32_t valid = (uint32_t)((n - tile_base < TILE) ? (n - tile_base) : TILE);
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  const uint32_t lane_off = wave * WAVE_SPAN + lane * VEC;  // + j*64*VEC per chunk

  // ---- load (elements past the end stand behind every real element of the tile, so whatever
  // they hold never reaches a result that is written)
  Vec16<T> x[CHUNKS];
  if (valid == TILE) {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) x[j] = load_vec<ALIGNED>(in + tile_base + lane_off + j * (WAVE * VEC));
  } else {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint32_t e = lane_off + j * (WAVE * VEC) + i;
        x[j].v[i] = (e < valid) ? in[tile_base + e] : T{};
      }
    }
  }

  // ---- wave-local scan in place, chunk by chunk: every element becomes the fold of the wave's
  // span up to it (inclusive), or up to but excluding it (exclusive; the span's very first
  // element has nothing before it and is fixed up with the prefix below)
  T carry = T{};  // fold of this wave's chunks before chunk j (j > 0)
#pragma unroll
  for (int j = 0; j < CHUNKS; ++j) {
    T s = x[j].v[0];
#pragma unroll
    for (int i = 1; i < VEC; ++i) s = op(s, x[j].v[i]);
    const T incl = wave_inclusive_scan_ordered(s, op, lane);
    const T before = dpp_move<0x138 /* wave_shr:1 */>(incl, incl);  // lane 0: unused
    const T chunk_total = readlane(incl, WAVE - 1);
    // fold of everything of the span before this lane's part of chunk j
    T run;
    bool has_run;
    if (j == 0) {
      run = before;
      has_run = lane > 0;
    } else {
      run = (lane == 0) ? carry : (T)op(carry, before);
      has_run = true;
    }
    carry = (j == 0) ? chunk_total : (T)op(carry, chunk_total);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const T e = x[j].v[i];
      const T with = (has_run || i > 0) ? (T)op(run, e) : e;
      if constexpr (EXCLUSIVE) x[j].v[i] = run;  // (lane 0 of chunk 0, i == 0: no meaning yet)
      else x[j].v[i] = with;
      run = with;
    }
  }
  if (lane == WAVE - 1) s_wave_agg[wave] = carry;  // the span's total (carry is wave-uniform)
  __syncthreads();
  T wave_prefix = T{};  // fold of the waves before this one (wave > 0)
  T block_agg = s_wave_agg[0];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) {
    if (w == wave) wave_prefix = block_agg;
    block_agg = op(block_agg, s_wave_agg[w]);
  }
  uint64_t* my_slot = status + (size_t)tile * W;

  // ---- cross-tile prefix
  if (wave == 0) {
    if (lane == 0) tile_publish<T>(my_slot, tile == 0 ? TS_INCLUSIVE : TS_PARTIAL, block_agg);
    if (tile != 0) {
      const T tile_excl = tile_lookback_ordered<T>(status, tile, op);
      if (lane == 0) {
        tile_publish<T>(my_slot, TS_INCLUSIVE, (T)op(tile_excl, block_agg));
        *s_prefix = tile_excl;
      }
    }
  }
  __syncthreads();
  // fold of everything before this wave's span: [init] [tiles before] [waves before], those that exist
  T prefix = init;
  bool has_prefix = EXCLUSIVE;
  if (tile != 0) {
    prefix = has_prefix ? (T)op(prefix, *s_prefix) : *s_prefix;
    has_prefix = true;
  }
  if (wave != 0) {
    prefix = has_prefix ? (T)op(prefix, wave_prefix) : wave_prefix;
    has_prefix = true;
  }

  // ---- apply the prefix and store
  if (has_prefix) {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        if (EXCLUSIVE && j == 0 && i == 0) x[j].v[i] = (lane == 0) ? prefix : (T)op(prefix, x[j].v[i]);
        else x[j].v[i] = op(prefix, x[j].v[i]);
      }
    }
  }
  if (valid == TILE) {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) store_vec<ALIGNED>(out + tile_base + lane_off + j * (WAVE * VEC), x[j]);
  } else {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint32_t e = lane_off + j * (WAVE * VEC) + i;
        if (e < valid) out[tile_base + e] = x[j].v[i];
      }
    }
  }
}

// Bytes of temporary storage for a scan of n elements of T: the ticket and the tile descriptors
// (sized for the small shape, which has the most tiles).
template <typename T>
inline size_t scan_temp_bytes(uint64_t n) {
  constexpr uint64_t TILE = (uint64_t)ScanShapeSmall::BLOCK * ScanShapeSmall::CHUNKS * Vec16<T>::N;
  const uint64_t tiles = (n + TILE - 1) / TILE;
  return 256 + align_up((size_t)tiles * TileWords<T>::W * sizeof(uint64_t), 256);
}

template <bool EXCLUSIVE, typename Shape, typename T, typename Op>
inline int ordered_scan_launch_shape(char* temp, const T* in, T* out, uint64_t n, T init, Op op, hipStream_t stream) {
  constexpr uint64_t TILE = (uint64_t)Shape::BLOCK * Shape::CHUNKS * Vec16<T>::N;
  const uint64_t tiles = (n + TILE - 1) / TILE;
  if (tiles > 0xffffffffull) return (int)hipErrorInvalidValue;
  uint32_t* ticket = reinterpret_cast<uint32_t*>(temp);
  uint64_t* status = reinterpret_cast<uint64_t*>(temp + 256);
  const uint64_t words = tiles * TileWords<T>::W;
  THRUST_AMD_KERNEL_LAUNCH("scan_init", stream, scan_init_kernel<0>, dim3((uint32_t)((words + 255) / 256)), dim3(256),
                           status, words, ticket);
  hipError_t e = hipPeekAtLastError();
  if (e != hipSuccess) return (int)e;
  if (is_aligned16(in) && is_aligned16(out))
    THRUST_AMD_KERNEL_LAUNCH("scan", stream, (ordered_scan_kernel<T, Op, EXCLUSIVE, true, Shape>), dim3((uint32_t)tiles),
                             dim3(Shape::BLOCK), in, out, n, init, op, status, ticket);
  else
    THRUST_AMD_KERNEL_LAUNCH("scan", stream, (ordered_scan_kernel<T, Op, EXCLUSIVE, false, Shape>), dim3((uint32_t)tiles),
                             dim3(Shape::BLOCK), in, out, n, init, op, status, ticket);
  return (int)hipPeekAtLastError();
}

// The scan of n > 0 elements; temp holds scan_temp_bytes<T>(n) bytes, 256-byte aligned.  out may be in.
template <bool EXCLUSIVE, typename T, typename Op>
inline int ordered_scan_launch(char* temp, const T* in, T* out, uint64_t n, T init, Op op, hipStream_t stream) {
  if (n * sizeof(T) >= SCAN_LARGE_MIN_BYTES)
    return ordered_scan_launch_shape<EXCLUSIVE, ScanShapeLarge>(temp, in, out, n, init, op, stream);
  return ordered_scan_launch_shape<EXCLUSIVE, ScanShapeSmall>(temp, in, out, n, init, op, stream);
}

}  // namespace scanning
}  // namespace hip
}  // namespace system
}  // namespace thrust
