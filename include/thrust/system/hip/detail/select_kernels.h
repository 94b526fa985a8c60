// The single-pass stream compaction kernel behind copy_if, remove_if, partition_copy,
// stable_partition, unique and unique_by_key, as templates on what decides the flags.
// libthrust_amd.so instantiates them for the comparison codes of its C interface
// (thrust_amd_copy_if, thrust_amd_partition_copy, thrust_amd_stable_partition,
// thrust_amd_unique, thrust_amd_unique_by_key); a translation unit compiled with hipcc
// instantiates them for its own predicates and key equalities, which then run inside the
// same kernel, as the reference passes the functor into its agents.
//
// One single-pass kernel serves all of them.  Every element gets a 0/1 flag
//   PRED   test(tested[i])                             (copy_if / partition: on the data itself,
//                                                       or on a stencil with the items as payload)
//   HEAD   i == 0 || test(tested[i-1], tested[i])      (unique, unique_by_key: test = "differ")
//   BYTE   tested[i] != 0, tested = uint8 flag array   (the library's stencil forms, after a flagging pass)
// and the exclusive prefix sum of the flags -- inside the lane, then across the wave with
// DPP, across the waves through LDS, across tiles by decoupled look-back with a dynamic
// tile ticket -- is the output position of each selected element; a rejected element goes
// to (its index - selected before it) of the second output when there is one.  The selected
// elements of a wave are contiguous in the output (and so are its rejected ones); each wave
// compacts them in its own piece of LDS first, so that its store instructions cover
// contiguous addresses.
//
// The in-place partition parks one side in temp storage and copies it back afterwards.  Its
// init kernel samples the input and picks the direction of the sweep so that the parked side
// is the smaller one: forwards, the selected elements are written in place (each lands at or
// before its source) and the rejected ones are parked; from the back, the rejected elements
// are written in place (each lands at or behind its source) and the selected ones are parked.
// Bytes moved: 8n + 8 min(selected, rejected) instead of 8n + 8 rejected.
//
// Outputs may alias inputs where the header says so: a tile learns its output offset
// only after every earlier tile has published its count, and a tile publishes only after
// all of its own loads have returned (explicit vmcnt(0) wait before the first barrier).
//
// HBM traffic: n*(tested + payload) read, selected (+ rejected) elements written,
// 16 bytes of tile descriptor per tile.  Replaces the CopyIfAgent / PartitionAgent /
// UniqueAgent / UniqueByKeyAgent kernels of the reference
// (thrust/system/cuda/detail/copy_if.h:365-478, partition.h:221-293, unique.h:316-445,
// unique_by_key.h:348-510).
//
// A Flagger says how flags are made.  It has one member,
//   template <typename Body> __device__ void per_tile(Body&& body) const
// which calls body(test, flip) once: `test(x)` (or, for head flags, `test(previous, x)`: x
// starts a run) gives an element's flag, `flip` (uniform) inverts every flag.  A flagger
// that chooses among several tests at run time branches once here, not once per element.
#pragma once
#include "device_primitives.h"

namespace thrust {
namespace system {
namespace hip {
namespace select {
using namespace ::thrust::system::hip::prim;

#define THRUST_AMD_SELECT_CHECK(expr)                \
  do {                                               \
    hipError_t _e = (expr);                          \
    if (_e != hipSuccess) return (int)_e;            \
  } while (0)

enum SelectFlagMode { FLAG_PRED = 0, FLAG_HEAD = 1, FLAG_BYTE = 2 };

// Two shapes.  What bounds this kernel is not arithmetic but how many bytes a CU holds while
// its tiles wait for their prefix: a tile stays in registers from its load until every earlier
// tile has published its count, and the memory system is only busy while loads are in flight.
// Measured on 2^28 float32 (copy_if at 50 % / 5 %): 1024 threads x 16 elements, two workgroups
// per CU (64 registers): 0.43 / 0.36 ms; 512 threads x 64 elements, two workgroups per CU
// (128 registers, twice the bytes per CU): 0.38 / 0.31 ms; 32 or 48 elements, three or four
// smaller workgroups per CU, 1024 x 32..64: all slower.  So: without a payload and with
// elements of up to four bytes, 512 threads x 64 elements (56 in the head-flag form, whose
// previous-element compare needs a few registers more: unique of 2^28 int32 0.39 -> 0.28 ms).
// With a payload, 1024 threads and 256 bytes of input per lane (at most 32 elements: narrow
// elements are unpacked into a register each), one workgroup per CU: unique_by_key of
// int32 + float32 0.54 -> 0.50 ms against 192 bytes per lane.
constexpr int SELECT_BLOCK = 1024;       // with a payload
constexpr int SELECT_LEAN_BLOCK = 512;   // without
constexpr int SELECT_LEAN_ITEMS = 64;
constexpr int SELECT_LEAN_HEAD_ITEMS = 56;
constexpr int SELECT_LEAN_TWO_ITEMS = 48;
constexpr int SELECT_LANE_BYTES = 256;
constexpr int SELECT_MIN_ITEMS = 8;   // sizes the descriptor array
constexpr int SELECT_MAX_ITEMS = 32;

// TWO: the kernel writes the rejected elements as well (partition).  Every element then goes
// through the LDS write-out; 48 elements per lane measured best there (the two-output kernel on
// 2^28 float32: 0.50 ms with 1024 threads x 16 elements, 0.46 ms with 512 x 48, 0.45-0.49 ms
// with 512 x 64).
template <typename T, typename U, bool HAS_PAYLOAD, int MODE, bool TWO = false>
struct SelectShape {
  static constexpr int VEC = Vec16<T>::N;
  static constexpr bool LEAN = !HAS_PAYLOAD && sizeof(T) <= 4;
  static constexpr bool LEAN_TWO = LEAN && TWO;
  static constexpr int BLOCK = LEAN ? SELECT_LEAN_BLOCK : SELECT_BLOCK;
  static constexpr int WAVES_PER_SIMD = 4;  // 128 registers: two lean workgroups per CU, or one with a payload
  // registers count, not bytes: an element narrower than four bytes still takes a register once unpacked
  static constexpr int BY_BYTES = SELECT_LANE_BYTES / (int)((sizeof(T) < 4 ? 4 : sizeof(T)) + (HAS_PAYLOAD ? (sizeof(U) < 4 ? 4 : sizeof(U)) : 0));
  // 8-byte elements without a payload: 24 instead of 32 (16 vectors' worth of flags and ranks beside
  // 64 data registers and 64-bit comparisons spilled)
  static constexpr int WIDE_ALONE = (!HAS_PAYLOAD && sizeof(T) == 8) ? 24 : SELECT_MAX_ITEMS;
  static constexpr int WANTED =
      LEAN_TWO ? SELECT_LEAN_TWO_ITEMS : LEAN ? (MODE == FLAG_HEAD ? SELECT_LEAN_HEAD_ITEMS : SELECT_LEAN_ITEMS)
           : (BY_BYTES < SELECT_MIN_ITEMS ? SELECT_MIN_ITEMS : (BY_BYTES > WIDE_ALONE ? WIDE_ALONE : BY_BYTES));
  static constexpr int CHUNKS = WANTED / VEC >= 1 ? WANTED / VEC : 1;
  static constexpr uint32_t TILE = (uint32_t)BLOCK * CHUNKS * VEC;
  // LDS of one wave for the write-out (at least one chunk of the payload).  All waves' regions
  // together also hold what a tile keeps while it waits for its prefix (see select_tile), so they
  // are as large as the CU allows: two lean workgroups of 72 KiB, or one of 128 KiB with a payload.
  static constexpr uint32_t PAYLOAD_CHUNK_BYTES = HAS_PAYLOAD ? (uint32_t)(WAVE * VEC * sizeof(U)) : 0u;
  // (copy_if of 2^28 float32 at 50 %: 0.328 ms with 4 KiB per wave, where only tiles that keep
  // less than a quarter are gathered, 0.312 ms with 9 KiB)
  static constexpr uint32_t WANTED_STAGE = LEAN ? 9216u : 8192u;
  static constexpr uint32_t STAGE_BYTES = PAYLOAD_CHUNK_BYTES > WANTED_STAGE ? PAYLOAD_CHUNK_BYTES : WANTED_STAGE;
};

// Write-out of one stream of a wave through the wave's own LDS region.  The wave's
// elements are handled in groups of G chunks: every lane drops its selected elements at
// their rank inside the group and (when there is a second output) its rejected elements
// behind them, in order; then consecutive lanes read consecutive slots, so that every
// store instruction covers one contiguous piece of the output.  The region is private to
// the wave and LDS executes a wave's instructions in order, so no barrier is needed
// between the two steps, only a compiler fence.
//   chunk_base[j]  selected elements of the wave before chunk j (wave-uniform)
//   lane_excl[j]   selected elements of the wave before this lane's part of chunk j
//   wave_valid     elements of the wave's span that exist (ragged last tile)
//   out_true       where the wave's first selected element goes
//   out_false      where the wave's first rejected element goes, or nullptr
//   rev            (wave-uniform) the outputs grow towards lower addresses: element k of a stream goes to out[-k]
template <bool HAS_FALSE, int CHUNKS, int VEC, int G, typename S, typename Get>
THRUST_AMD_DEVICE void select_emit(const bool rev, S* stage, const uint32_t (&fl)[CHUNKS], const uint32_t (&lane_excl)[CHUNKS],
                           const uint32_t (&chunk_base)[CHUNKS + 1], int lane, uint32_t wave_valid,
                           S* out_true, S* out_false, Get get) {
  constexpr uint32_t CHUNK_ELEMS = WAVE * VEC;
#pragma unroll
  for (int g0 = 0; g0 < CHUNKS; g0 += G) {
    const int ge = (CHUNKS - g0 < G) ? CHUNKS - g0 : G;
    const uint32_t sel0 = chunk_base[g0];
    const uint32_t sel_g = chunk_base[g0 + ge] - sel0;
    const uint32_t e0 = (uint32_t)g0 * CHUNK_ELEMS;
    const uint32_t left = wave_valid > e0 ? wave_valid - e0 : 0u;
    const uint32_t e_cnt = left < (uint32_t)ge * CHUNK_ELEMS ? left : (uint32_t)ge * CHUNK_ELEMS;
#pragma unroll
    for (int jj = 0; jj < G; ++jj) {
      const int j = g0 + jj;
      if (j < CHUNKS) {
        uint32_t r = lane_excl[j] - sel0;
        // slot of a rejected element = sel_g + (its offset in the group) - (selected before it)
        uint32_t rej = sel_g + (uint32_t)jj * CHUNK_ELEMS + (uint32_t)lane * VEC - r;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const bool sel = (fl[j] >> i) & 1u;
          if constexpr (HAS_FALSE) {
            const uint32_t e = (uint32_t)jj * CHUNK_ELEMS + (uint32_t)lane * VEC + i;
            if (sel || e < e_cnt) stage[sel ? r : rej] = get(j, i);
            rej += sel ? 0u : 1u;
          } else {
            if (sel) stage[r] = get(j, i);
          }
          r += sel ? 1u : 0u;
        }
      }
    }
    asm volatile("" ::: "memory");
    const uint32_t limit = HAS_FALSE ? e_cnt : sel_g;
    if (HAS_FALSE && rev) {
      for (uint32_t slot = lane; slot < limit; slot += WAVE) {
        const S v = stage[slot];
        if (slot < sel_g) *(out_true - (sel0 + slot)) = v;
        else *(out_false - ((e0 - sel0) + (slot - sel_g))) = v;
      }
    } else {
      for (uint32_t slot = lane; slot < limit; slot += WAVE) {
        const S v = stage[slot];
        if (!HAS_FALSE || slot < sel_g) out_true[sel0 + slot] = v;
        else out_false[(e0 - sel0) + (slot - sel_g)] = v;
      }
    }
    asm volatile("" ::: "memory");
  }
}

template <typename T, typename U, typename Flagger>
struct SelectArgs {
  const T* tested;      // array the flags come from
  const U* payload;     // second stream compacted with the same flags (or nullptr)
  T* tested_true;       // selected tested elements (nullptr: not emitted)
  T* tested_false;      // rejected tested elements (nullptr: not emitted)
  U* payload_true;
  U* payload_false;
  uint64_t* d_num_true;
  uint64_t n;
  Flagger flag;         // how an element's flag is made
  uint64_t* status;
  uint32_t* ticket;
  uint32_t aligned;     // tested (and payload) pointers allow whole-vector loads
  const uint32_t* reverse;  // in-place partition only: *reverse != 0 sweeps from the back (else nullptr)
};

// Arguments with every pointer null and the given flagger (which need not be default-constructible).
template <typename T, typename U, typename Flagger>
inline SelectArgs<T, U, Flagger> make_select_args(const Flagger& flag) {
  return SelectArgs<T, U, Flagger>{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0,
                                   flag,    nullptr, nullptr, 0u,      nullptr};
}

// VEC elements of U that belong to one 16-byte vector of T.
template <typename U, int VEC>
struct alignas((VEC * sizeof(U)) >= 16 ? 16 : VEC * sizeof(U)) PayloadVec {
  U v[VEC];
};

// Clears the tile descriptors, the ticket and the count.  For the in-place partition it also
// decides the direction of the sweep from a sample of the input (workgroup 0: 4096 elements
// spread evenly): the side the sample finds smaller is the one that gets parked in temporary
// storage and copied back.  Whatever the sample says, both directions give the same result.
template <typename T, int MODE, typename Flagger>
__global__ __launch_bounds__(256) void select_init_kernel(uint64_t* __restrict__ words,
                                                          uint64_t count,
                                                          uint32_t* __restrict__ ticket,
                                                          uint64_t* __restrict__ d_num,
                                                          const T* __restrict__ tested, uint64_t n,
                                                          Flagger flag,
                                                          uint32_t* __restrict__ reverse) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) words[i] = 0;
  if (i == 0) {
    *ticket = 0;
    *d_num = 0;
  }
  if (reverse != nullptr && blockIdx.x == 0) {
    constexpr int PER_LANE = 16;
    __shared__ uint32_t s_hits;
    if (threadIdx.x == 0) s_hits = 0;
    __syncthreads();
    const uint64_t samples = (uint64_t)256 * PER_LANE;
    const uint64_t step = n / samples ? n / samples : 1;
    uint32_t hits = 0, seen = 0;
    if constexpr (MODE != FLAG_HEAD) {
      flag.per_tile([&](auto test, bool flip) {
#pragma unroll
        for (int k = 0; k < PER_LANE; ++k) {
          const uint64_t idx = ((uint64_t)k * 256 + threadIdx.x) * step;
          if (idx < n) {
            const T x = tested[idx];
            hits += ((bool)test(x) != flip) ? 1u : 0u;
            ++seen;
          }
        }
      });
    }
    atomicAdd(&s_hits, (hits << 16) | seen);  // at most 4096 of each: no carry between the halves
    __syncthreads();
    if (threadIdx.x == 0) {
      const uint32_t h = s_hits >> 16, c = s_hits & 0xffffu;
      *reverse = (2 * h < c) ? 1u : 0u;  // few selected: park them, write the rejected in place
    }
  }
}

// Shared memory of one workgroup of the selection kernel.
template <typename T, typename U, int MODE, bool HAS_PAYLOAD, bool TWO>
struct SelectShared {
  using Shape = SelectShape<T, U, HAS_PAYLOAD, MODE, TWO>;
  uint32_t tile;
  uint32_t wave_cnt[Shape::BLOCK / WAVE];
  uint64_t prefix;
  __attribute__((aligned(16))) unsigned char stage[(size_t)(Shape::BLOCK / WAVE) * Shape::STAGE_BYTES];
};

// One tile.  REV = the sweep runs from the back of the input: tile 0 is the last tile in memory
// and "element k" of the tile (and of every output stream) is counted from the back, so the
// same ranks serve; a lane's vectors are loaded from the mirrored address and their elements
// swapped end for end.  Only the in-place partition uses it.
template <typename T, typename U, int MODE, bool HAS_PAYLOAD, bool TWO, bool REV, typename Flagger>
THRUST_AMD_DEVICE void select_tile(const SelectArgs<T, U, Flagger>& a, SelectShared<T, U, MODE, HAS_PAYLOAD, TWO>& sh) {
  using Shape = SelectShape<T, U, HAS_PAYLOAD, MODE, TWO>;
  constexpr int VEC = Shape::VEC;
  constexpr int CHUNKS = Shape::CHUNKS;
  constexpr int WAVES = Shape::BLOCK / WAVE;
  constexpr uint32_t WAVE_SPAN = WAVE * CHUNKS * VEC;
  constexpr uint32_t TILE = Shape::TILE;
  using PV = PayloadVec<U, VEC>;
  static_assert(!(REV && MODE == FLAG_HEAD), "head flags are only formed front to back");

  const uint32_t tile = sh.tile;
  const uint64_t tiles_total = (a.n + TILE - 1) / TILE;
  // the tile's place in memory, and the number of elements that come before it in sweep order
  const uint64_t mem_base = (REV ? (tiles_total - 1 - tile) : (uint64_t)tile) * TILE;
  const uint32_t valid = (uint32_t)((a.n - mem_base < TILE) ? (a.n - mem_base) : TILE);
  const uint64_t tile_base = REV ? a.n - mem_base - valid : mem_base;
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  const uint32_t lane_off = wave * WAVE_SPAN + lane * VEC;  // + j*64*VEC
  const bool full = valid == TILE;
  // memory index of the tile's element e (in sweep order)
  auto mem_index = [&](uint32_t e) -> uint64_t { return REV ? mem_base + (valid - 1 - e) : mem_base + e; };

  // ---- load
  T wave_prev = T{};
  if constexpr (MODE == FLAG_HEAD) {
    // every lane reads the one element before the wave's span, unconditionally, so that
    // this load is in flight together with the tile's
    const uint64_t first = tile_base + (uint64_t)wave * WAVE_SPAN;
    wave_prev = a.tested[(first > 0 && first < a.n) ? first - 1 : 0];
  }
  Vec16<T> x[CHUNKS];
  PV y[HAS_PAYLOAD ? CHUNKS : 1];
  if (full && a.aligned) {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const uint32_t e0 = lane_off + j * (WAVE * VEC);
      const uint64_t off = REV ? mem_base + (TILE - VEC - e0) : mem_base + e0;
      x[j] = *reinterpret_cast<const Vec16<T>*>(a.tested + off);
      if constexpr (HAS_PAYLOAD) y[j] = *reinterpret_cast<const PV*>(a.payload + off);
    }
    if constexpr (REV) {
#pragma unroll
      for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
        for (int i = 0; i < VEC / 2; ++i) {
          const T t = x[j].v[i];
          x[j].v[i] = x[j].v[VEC - 1 - i];
          x[j].v[VEC - 1 - i] = t;
          if constexpr (HAS_PAYLOAD) {
            const U u = y[j].v[i];
            y[j].v[i] = y[j].v[VEC - 1 - i];
            y[j].v[VEC - 1 - i] = u;
          }
        }
      }
    }
  } else if (full) {
    // pointers that do not allow whole vectors: element loads, still without predicates
    // (a predicated load makes the compiler wait for it before issuing the next one)
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint64_t off = mem_index(lane_off + j * (WAVE * VEC) + i);
        x[j].v[i] = a.tested[off];
        if constexpr (HAS_PAYLOAD) y[j].v[i] = a.payload[off];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint32_t e = lane_off + j * (WAVE * VEC) + i;
        x[j].v[i] = (e < valid) ? a.tested[mem_index(e)] : T{};
        if constexpr (HAS_PAYLOAD) y[j].v[i] = (e < valid) ? a.payload[mem_index(e)] : U{};
      }
    }
  }

  // ---- flags (bit i of fl[j] = element i of chunk j is selected)
  uint32_t fl[CHUNKS];
  a.flag.per_tile([&](auto test, bool flip) {
    if constexpr (MODE == FLAG_HEAD) {
#pragma unroll
      for (int j = 0; j < CHUNKS; ++j) {
        // predecessor of the lane's first element: last element of the previous lane; for
        // lane 0 the last element of the previous chunk (lane 63 holds it) or, for the first
        // chunk, the element just before the wave's span, loaded with the tile
        T prev = dpp_move<0x138 /* wave_shr:1 */>(x[j].v[VEC - 1], x[j].v[VEC - 1]);
        const T before = (j == 0) ? wave_prev : readlane(x[j > 0 ? j - 1 : 0].v[VEC - 1], WAVE - 1);
        const uint64_t first = tile_base + lane_off + j * (WAVE * VEC);
        bool head0 = false;
        if (lane == 0) {
          if (first == 0) head0 = true;
          else prev = before;
        }
        uint32_t f = 0;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          bool h = (bool)test((i == 0) ? prev : x[j].v[i > 0 ? i - 1 : 0], x[j].v[i]);
          if (i == 0) h = h || head0;
          f |= (uint32_t)h << i;
        }
        fl[j] = f;
      }
    } else {
      const uint32_t flip_mask = flip ? ((1u << VEC) - 1u) : 0u;
#pragma unroll
      for (int j = 0; j < CHUNKS; ++j) {
        uint32_t f = 0;
#pragma unroll
        for (int i = 0; i < VEC; ++i) f |= (uint32_t)(bool)test(x[j].v[i]) << i;
        fl[j] = f ^ flip_mask;
      }
    }
  });
  if (!full) {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const uint32_t e0 = lane_off + j * (WAVE * VEC);
      const uint32_t live = (e0 >= valid) ? 0u : ((valid - e0 >= (uint32_t)VEC) ? ((1u << VEC) - 1u) : ((1u << (valid - e0)) - 1u));
      fl[j] &= live;
    }
  }

  // ---- ranks: lane -> wave (DPP scans chained over the chunks) -> workgroup
  uint32_t lane_excl[CHUNKS];
  uint32_t chunk_base[CHUNKS + 1];  // wave-uniform
  chunk_base[0] = 0;
#pragma unroll
  for (int j = 0; j < CHUNKS; ++j) {
    const uint32_t c = __builtin_popcount(fl[j]);
    const uint32_t incl = wave_inclusive_scan(c, OpPlus{});
    lane_excl[j] = chunk_base[j] + dpp_move<0x138>(0u, incl);
    chunk_base[j + 1] = chunk_base[j] + readlane(incl, WAVE - 1);
  }
  if (lane == 0) sh.wave_cnt[wave] = chunk_base[CHUNKS];
  // every load of this wave has returned before the tile's count can become visible:
  // in-place callers rely on it (see the file comment)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  uint32_t wave_prefix = 0, tile_cnt = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    if (w == wave) wave_prefix = tile_cnt;
    tile_cnt += sh.wave_cnt[w];
  }

  // ---- selected elements before this tile
  constexpr int W = TileWords<uint64_t>::W;
  uint64_t* my_slot = a.status + (size_t)tile * W;
  if (wave == 0 && lane == 0) tile_publish<uint64_t>(my_slot, tile == 0 ? TS_INCLUSIVE : TS_PARTIAL, (uint64_t)tile_cnt);

  // A tile that keeps few elements (one output, forward sweep) gathers them in LDS at their place
  // inside the tile while its prefix is on its way, and has only a coalesced copy left to do when
  // it arrives.  The workgroup's write-out regions together serve as the gathering area.
  constexpr uint32_t STAGE_TOTAL = (uint32_t)WAVES * Shape::STAGE_BYTES;
  // (a multiple of 16 elements, so that the payload's part starts on a 16-byte boundary)
  constexpr uint32_t GATHER_CAP = (STAGE_TOTAL / (uint32_t)(sizeof(T) + (HAS_PAYLOAD ? sizeof(U) : 0))) & ~15u;
  T* gather_tested = reinterpret_cast<T*>(sh.stage);
  U* gather_payload = reinterpret_cast<U*>(sh.stage + (size_t)GATHER_CAP * sizeof(T));
  const bool gathered = !TWO && !REV && tile_cnt <= GATHER_CAP;
  if constexpr (!TWO && !REV) {
    if (gathered) {
#pragma unroll
      for (int j = 0; j < CHUNKS; ++j) {
        uint32_t r = wave_prefix + lane_excl[j];
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          if ((fl[j] >> i) & 1u) {
            if (a.tested_true) gather_tested[r] = x[j].v[i];
            if constexpr (HAS_PAYLOAD) gather_payload[r] = y[j].v[i];
            ++r;
          }
        }
      }
    }
  }

  if (wave == 0) {
    uint64_t excl = 0;
    if (tile != 0) {
      excl = tile_lookback<uint64_t>(a.status, tile, OpPlus{}, (uint64_t)0);
      if (lane == 0) tile_publish<uint64_t>(my_slot, TS_INCLUSIVE, excl + tile_cnt);
    }
    if (lane == 0) {
      sh.prefix = excl;
      if ((uint64_t)tile + 1 == tiles_total) *a.d_num_true = excl + tile_cnt;
    }
  }
  __syncthreads();
  if constexpr (!TWO && !REV) {
    if (gathered) {
      const uint64_t base = sh.prefix;
      if (a.tested_true)
        for (uint32_t e = threadIdx.x; e < tile_cnt; e += Shape::BLOCK) a.tested_true[base + e] = gather_tested[e];
      if constexpr (HAS_PAYLOAD)
        for (uint32_t e = threadIdx.x; e < tile_cnt; e += Shape::BLOCK) a.payload_true[base + e] = gather_payload[e];
      return;
    }
  }
  // the wave's selected elements start at prefix + wave_prefix of the first output; a
  // rejected element at tile offset e with r selected elements before it in the tile
  // lands at (tile_base - prefix) + e - r of the second output
  const uint64_t true_base = sh.prefix + wave_prefix;
  const uint32_t wave_e0 = (uint32_t)wave * WAVE_SPAN;
  const uint64_t false_base = tile_base - sh.prefix + wave_e0 - wave_prefix;
  const uint32_t wave_valid = valid > wave_e0 ? (valid - wave_e0 < WAVE_SPAN ? valid - wave_e0 : WAVE_SPAN) : 0u;

  // ---- write-out
  // Forward: stream k of an output goes to out[k].  From the back (in-place partition):
  // the selected elements are the parked ones, stream element k goes to parked[n-1-k], and
  // the rejected ones go in place to data[n-1-k]; the roles of the two buffers are swapped.
  auto emit = [&](auto* fwd_true, auto* fwd_false, auto get) {
    using S = std::remove_pointer_t<decltype(fwd_true)>;
    constexpr int G = (int)(Shape::STAGE_BYTES / (WAVE * VEC * sizeof(S)));
    S* stage = reinterpret_cast<S*>(sh.stage + (size_t)wave * Shape::STAGE_BYTES);
    if constexpr (REV) {
      S* out_true = fwd_false + (a.n - 1) - true_base;
      S* out_false = fwd_true + (a.n - 1) - false_base;
      select_emit<true, CHUNKS, VEC, G>(true, stage, fl, lane_excl, chunk_base, lane, wave_valid, out_true, out_false, get);
    } else {
      S* out_true = fwd_true + true_base;
      if (fwd_false)
        select_emit<true, CHUNKS, VEC, G>(false, stage, fl, lane_excl, chunk_base, lane, wave_valid, out_true, fwd_false + false_base, get);
      else
        select_emit<false, CHUNKS, VEC, G>(false, stage, fl, lane_excl, chunk_base, lane, wave_valid, out_true, (S*)nullptr, get);
    }
  };
  if (a.tested_true) emit(a.tested_true, a.tested_false, [&](int j, int i) { return x[j].v[i]; });
  if constexpr (HAS_PAYLOAD) emit(a.payload_true, a.payload_false, [&](int j, int i) { return y[j].v[i]; });
}

// DIR 0: forward sweep.  DIR 1 / 2: the two kernels of the in-place partition, launched one
// after the other; the one whose direction (1 forward, 2 from the back) the init kernel did not
// choose ends at once.  (One kernel that takes the direction as a run-time value, or that
// holds both bodies, was measured at twice the time: 0.9 against 0.5 ms on 2^28 float32.)
template <typename T, typename U, int MODE, bool HAS_PAYLOAD, bool TWO, int DIR, typename Flagger>
__global__ __launch_bounds__((SelectShape<T, U, HAS_PAYLOAD, MODE, TWO>::BLOCK), (SelectShape<T, U, HAS_PAYLOAD, MODE, TWO>::WAVES_PER_SIMD))
void select_kernel(SelectArgs<T, U, Flagger> a) {
  if constexpr (DIR != 0) {
    if ((*a.reverse != 0) != (DIR == 2)) return;
  }
  __shared__ SelectShared<T, U, MODE, HAS_PAYLOAD, TWO> sh;
  if (threadIdx.x == 0) sh.tile = atomicAdd(a.ticket, 1u);
  __syncthreads();
  select_tile<T, U, MODE, HAS_PAYLOAD, TWO, DIR == 2>(a, sh);
}


// Second step of the in-place partition: the parked elements move to their place.  After a
// forward sweep these are the rejected ones, parked[0, F) -> data[T, n); after a sweep from
// the back the selected ones, parked[n - T, n) -> data[0, T).
// 16-byte loads on the source's grid and 16-byte stores on the destination's: the two grids
// differ by H elements (the same H everywhere), so a destination vector is put together from
// two neighbouring source vectors.  (16-byte stores fed by loads that are only
// element-aligned were measured slower than plain element copies.)
constexpr int TAIL_BLOCK = 256;
constexpr int TAIL_UNROLL = 8;         // destination vectors per lane
constexpr int TAIL_UNROLL_NARROW = 2;  // the same for items of 1 or 2 bytes, which are copied element by element

// One workgroup moves TAIL_BLOCK * TAIL_UNROLL destination vectors and ends: many short
// workgroups keep more loads in flight than a few long-running ones (a grid-stride loop
// over the same copy reached 4.5 TB/s).  The grid is sized for n elements, because the host
// does not know how many are parked; a workgroup with nothing to move still costs its launch
// and two scalar loads, and with 2 vectors per lane the empty ones alone took 60 us at
// 2^28 four-byte items (stable_partition with 5 % selected: 0.533 ms; 4 vectors 0.506, 8 vectors
// 0.490, 16 vectors 0.491).  src_aligned[j] and src_aligned[j + 1] together hold
// destination vector j, starting at element H of the first.
template <typename U, int H>
THRUST_AMD_DEVICE void partition_tail_vectors(U* __restrict__ dst_aligned, const U* __restrict__ src_aligned, uint64_t vecs) {
  constexpr int VEC = Vec16<U>::N;
  const Vec16<U>* src = reinterpret_cast<const Vec16<U>*>(src_aligned);
  Vec16<U>* out = reinterpret_cast<Vec16<U>*>(dst_aligned);
  const uint64_t base = (uint64_t)blockIdx.x * (TAIL_BLOCK * TAIL_UNROLL) + threadIdx.x;
  if (base >= vecs) return;
  Vec16<U> lo[TAIL_UNROLL], hi[TAIL_UNROLL];
  if (base + (TAIL_UNROLL - 1) * TAIL_BLOCK < vecs) {
#pragma unroll
    for (int u = 0; u < TAIL_UNROLL; ++u) {
      lo[u] = src[base + u * TAIL_BLOCK];
      if (H != 0) hi[u] = src[base + u * TAIL_BLOCK + 1];
    }
  } else {
#pragma unroll
    for (int u = 0; u < TAIL_UNROLL; ++u) {
      if (base + u * TAIL_BLOCK < vecs) {
        lo[u] = src[base + u * TAIL_BLOCK];
        if (H != 0) hi[u] = src[base + u * TAIL_BLOCK + 1];
      }
    }
  }
#pragma unroll
  for (int u = 0; u < TAIL_UNROLL; ++u) {
    if (base + u * TAIL_BLOCK < vecs) {
      Vec16<U> o;
#pragma unroll
      for (int k = 0; k < VEC; ++k) o.v[k] = (H + k < VEC) ? lo[u].v[(H + k) % VEC] : hi[u].v[(H + k) % VEC];
      out[base + u * TAIL_BLOCK] = o;
    }
  }
}

// Launched with enough workgroups for n elements; those past the parked count end at once.
template <typename U>
__global__ __launch_bounds__(TAIL_BLOCK) void partition_tail_kernel(U* __restrict__ data,
                                                                    const U* __restrict__ parked,
                                                                    uint64_t n,
                                                                    const uint64_t* __restrict__ d_num_true,
                                                                    const uint32_t* __restrict__ reverse) {
  const uint64_t t = *d_num_true;
  const bool rev = *reverse != 0;
  const uint64_t f = rev ? t : n - t;               // elements to move
  U* dst = rev ? data : data + t;
  const U* src = rev ? parked + (n - t) : parked;
  constexpr int VEC = Vec16<U>::N;
  const uint64_t gid = (uint64_t)blockIdx.x * TAIL_BLOCK + threadIdx.x;
  if constexpr (sizeof(U) >= 4) {
    // destination element `head` is the first on a 16-byte boundary; destination vector j holds
    // src[head + j*VEC ...], which starts H elements into an aligned source vector
    uint64_t head = ((16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15) / sizeof(U);
    if (head > f) head = f;
    const U* s0 = src + head;
    const int h = (int)((reinterpret_cast<uintptr_t>(s0) & 15) / sizeof(U));
    uint64_t vecs = (f - head) / VEC;
    // the second source vector of the last destination vector must lie inside src[0, f)
    if (h != 0 && vecs != 0 && head + vecs * VEC + (VEC - h) > f) vecs -= 1;
    switch (h) {
      case 0: partition_tail_vectors<U, 0>(dst + head, s0, vecs); break;
      case 1: partition_tail_vectors<U, 1 % VEC>(dst + head, s0 - 1, vecs); break;
      case 2: partition_tail_vectors<U, 2 % VEC>(dst + head, s0 - 2, vecs); break;
      default: partition_tail_vectors<U, 3 % VEC>(dst + head, s0 - 3, vecs); break;
    }
    // the elements before the first and after the last whole vector (fewer than 3 * VEC)
    if (gid < head) dst[gid] = src[gid];
    const uint64_t done = head + vecs * VEC;
    if (done + gid < f) dst[done + gid] = src[done + gid];
  } else {
    // narrow items: element copies, TAIL_UNROLL_NARROW * VEC per lane
    const uint64_t base = (uint64_t)blockIdx.x * (TAIL_BLOCK * TAIL_UNROLL_NARROW * VEC) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < TAIL_UNROLL_NARROW * VEC; ++u) {
      const uint64_t i = base + (uint64_t)u * TAIL_BLOCK;
      if (i < f) dst[i] = src[i];
    }
  }
}

struct SelectTemp {
  size_t off_ticket, off_status, off_extra, total;
  uint64_t tiles;
};

// Sized for the smallest tile any payload type leads to, so that the temp size does not
// depend on the payload; the launch uses the tile count of its own shape.
template <typename T>
inline SelectTemp select_layout(uint64_t n, size_t extra_bytes) {
  constexpr int VEC = Vec16<T>::N;
  constexpr uint64_t TILE = (uint64_t)SELECT_BLOCK * (VEC > SELECT_MIN_ITEMS ? VEC : SELECT_MIN_ITEMS);
  SelectTemp t;
  t.tiles = (n + TILE - 1) / TILE;
  TempLayout lay;
  t.off_ticket = lay.add(sizeof(uint32_t));
  t.off_status = lay.add((size_t)t.tiles * TileWords<uint64_t>::W * sizeof(uint64_t));
  t.off_extra = lay.add(extra_bytes);
  t.total = lay.total;
  return t;
}

// DUAL: the in-place partition; the init kernel picks the direction of the sweep and leaves it
// in temp storage (the word 64 bytes behind the ticket) for the kernels that follow: one
// selection kernel per direction, of which the other ends at once, and the copy back.
template <typename T, typename U, int MODE, bool HAS_PAYLOAD, bool TWO = false, bool DUAL = false, typename Flagger>
inline int select_launch(char* temp, const SelectTemp& lay, SelectArgs<T, U, Flagger> a, hipStream_t stream) {
  constexpr uint64_t TILE = SelectShape<T, U, HAS_PAYLOAD, MODE, TWO>::TILE;
  const uint64_t tiles = (a.n + TILE - 1) / TILE;
  if (tiles > 0xffffffffull || tiles > lay.tiles) return (int)hipErrorInvalidValue;
  a.ticket = reinterpret_cast<uint32_t*>(temp + lay.off_ticket);
  a.status = reinterpret_cast<uint64_t*>(temp + lay.off_status);
  uint32_t* reverse = DUAL ? a.ticket + 16 : nullptr;
  a.reverse = reverse;
  constexpr size_t PAY_ALIGN = alignof(PayloadVec<U, Vec16<T>::N>);
  a.aligned = is_aligned16(a.tested) &&
              (!HAS_PAYLOAD || (reinterpret_cast<uintptr_t>(a.payload) % PAY_ALIGN) == 0);
  const uint64_t words = tiles * TileWords<uint64_t>::W;
  const uint64_t init_threads = words ? words : 1;
  THRUST_AMD_KERNEL_LAUNCH("select_init", stream, (select_init_kernel<T, MODE, Flagger>),
                           dim3((uint32_t)((init_threads + 255) / 256)), dim3(256), a.status, words, a.ticket,
                           a.d_num_true, a.tested, a.n, a.flag, reverse);
  THRUST_AMD_SELECT_CHECK(hipPeekAtLastError());
  if (a.n == 0) return 0;
  if constexpr (DUAL) {
    THRUST_AMD_KERNEL_LAUNCH("select", stream, (select_kernel<T, U, MODE, HAS_PAYLOAD, TWO, 1, Flagger>), dim3((uint32_t)tiles),
              dim3(SelectShape<T, U, HAS_PAYLOAD, MODE, TWO>::BLOCK), a);
    THRUST_AMD_SELECT_CHECK(hipPeekAtLastError());
    THRUST_AMD_KERNEL_LAUNCH("select", stream, (select_kernel<T, U, MODE, HAS_PAYLOAD, TWO, 2, Flagger>), dim3((uint32_t)tiles),
              dim3(SelectShape<T, U, HAS_PAYLOAD, MODE, TWO>::BLOCK), a);
  } else {
    THRUST_AMD_KERNEL_LAUNCH("select", stream, (select_kernel<T, U, MODE, HAS_PAYLOAD, TWO, 0, Flagger>), dim3((uint32_t)tiles),
              dim3(SelectShape<T, U, HAS_PAYLOAD, MODE, TWO>::BLOCK), a);
  }
  THRUST_AMD_SELECT_CHECK(hipPeekAtLastError());
  return 0;
}

template <typename U>
inline uint32_t tail_grid(uint64_t n) {
  const uint64_t per_block = (uint64_t)TAIL_BLOCK * (sizeof(U) >= 4 ? TAIL_UNROLL : TAIL_UNROLL_NARROW) * Vec16<U>::N;
  return (uint32_t)((n + per_block - 1) / per_block + 1);
}


#undef THRUST_AMD_SELECT_CHECK

}  // namespace select
}  // namespace hip
}  // namespace system
}  // namespace thrust
