// What the memory system gives to a kernel that does nothing but the memory accesses of one
// pass of a least-significant-digit radix sort: every workgroup reads a tile of consecutive
// keys and writes it as 256 runs, one per digit value, each run behind the same digit's run of
// the tile before it.  No digits are extracted and nothing is ranked: element e of a tile simply
// goes to run e / RUN, so the kernel is a fixed permutation with exactly the write pattern of a
// pass over keys whose digits are uniform.  The library's pass (18432-key tiles, runs of 72 keys
// = 288 bytes) is measured against 8 TB/s; these kernels show how much of that any kernel
// with this write pattern reaches, and how the run length changes it.
// Standalone HIP program (does not use the library); checks that every variant is a permutation
// of the input, prints one line per kernel and PASSED when the figures are sane.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <vector>

#define CHECK(expr)                                                 \
  do {                                                              \
    hipError_t e_ = (expr);                                         \
    if (e_ != hipSuccess) {                                         \
      std::printf("%s failed: %s\n", #expr, hipGetErrorString(e_)); \
      return 1;                                                     \
    }                                                               \
  } while (0)

constexpr int BLOCK = 1024;
constexpr int ITEMS = 18;
constexpr uint32_t TILE = BLOCK * ITEMS;  // 18432 keys, the library's tile for 4-byte keys

// RUN keys per run (TILE / RUN runs per tile); RUN == TILE writes the tile where it was read.
// tiles * TILE == n, so run r of tile t starts at r * (n / (TILE / RUN)) + t * RUN and the
// last one ends at n.
// BY_XCD: workgroups are dealt to the 8 XCDs in turn (workgroup i runs on XCD i % 8); with it,
// every XCD takes a contiguous eighth of the tiles in order, so that the tile whose runs
// continue a tile's runs passes through the same L2.
template <uint32_t RUN, bool BY_XCD = false, int ITEMS = ::ITEMS>
__global__ __launch_bounds__(BLOCK) void pass_pattern(const uint32_t* __restrict__ in, uint32_t* __restrict__ out,
                                                      uint32_t tiles, uint32_t group) {
  constexpr uint32_t TILE = BLOCK * ITEMS;
  constexpr uint32_t RUNS = TILE / RUN;
  static_assert(TILE % RUN == 0, "whole runs");
  // BY_XCD: the workgroups of one XCD (blockIdx % 8) take `group` consecutive tiles, then the next
  // `group` tiles 8 groups further on
  const uint32_t x = blockIdx.x % 8, j = blockIdx.x / 8;
  const uint32_t tile = BY_XCD ? ((j / group) * 8 + x) * group + j % group : blockIdx.x;
  if (tile >= tiles) return;
  const uint32_t* src = in + (size_t)tile * TILE;
  const uint32_t per_run_region = tiles * RUN;  // keys of one run index over all tiles = n / RUNS
  uint32_t k[ITEMS];
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) k[r] = src[(uint32_t)r * BLOCK + threadIdx.x];
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    const uint32_t e = (uint32_t)r * BLOCK + threadIdx.x;  // < TILE
    const uint32_t run = e / RUN, within = e % RUN;        // run < RUNS
    out[(size_t)run * per_run_region + (size_t)tile * RUN + within] = k[r];
  }
  (void)RUNS;
}

// The same for pairs of a 64-bit key and a 32-bit value in the library's 8192-pair tiles: both
// arrays are written as TILE_P / RUN runs of RUN elements (a pass of 8-bit digits: 256 runs of 32).
constexpr int ITEMS_P = 8;
constexpr uint32_t TILE_P = BLOCK * ITEMS_P;
template <uint32_t RUN>
__global__ __launch_bounds__(BLOCK) void pass_pattern_pairs(const uint64_t* __restrict__ kin, uint64_t* __restrict__ kout,
                                                            const uint32_t* __restrict__ vin, uint32_t* __restrict__ vout,
                                                            uint32_t tiles) {
  static_assert(TILE_P % RUN == 0, "whole runs");
  const uint32_t tile = blockIdx.x;
  const uint64_t* ksrc = kin + (size_t)tile * TILE_P;
  const uint32_t* vsrc = vin + (size_t)tile * TILE_P;
  const uint32_t per_run_region = tiles * RUN;
  uint64_t k[ITEMS_P];
  uint32_t v[ITEMS_P];
#pragma unroll
  for (int r = 0; r < ITEMS_P; ++r) {
    k[r] = ksrc[(uint32_t)r * BLOCK + threadIdx.x];
    v[r] = vsrc[(uint32_t)r * BLOCK + threadIdx.x];
  }
#pragma unroll
  for (int r = 0; r < ITEMS_P; ++r) {
    const uint32_t e = (uint32_t)r * BLOCK + threadIdx.x;  // < TILE_P
    const size_t dst = (size_t)(e / RUN) * per_run_region + (size_t)tile * RUN + e % RUN;  // < tiles * TILE_P
    kout[dst] = k[r];
    vout[dst] = v[r];
  }
}

// sum and xor of all keys: equal for input and output when the output is a permutation of the input
__global__ void checksum(const uint32_t* __restrict__ p, size_t n, unsigned long long* sums) {
  unsigned long long s = 0, x = 0;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    s += p[i];
    x ^= (unsigned long long)p[i] * 0x9E3779B97F4A7C15ull;
  }
  atomicAdd(&sums[0], s);
  atomicXor(&sums[1], x);
}

int main() {
  const uint32_t tiles = 14563;           // 14563 * 18432 = 268 425 216 keys, just under 2^28
  const size_t n = (size_t)tiles * TILE;  // 4 n bytes per array: 1.0 GiB
  uint32_t *in = nullptr, *out = nullptr;
  unsigned long long* sums = nullptr;
  CHECK(hipMalloc(&in, n * 4));
  CHECK(hipMalloc(&out, n * 4));
  CHECK(hipMalloc(&sums, 4 * sizeof(unsigned long long)));
  {
    std::vector<uint32_t> h(n);
    uint64_t s = 0x243F6A8885A308D3ull;
    for (size_t i = 0; i < n; ++i) {
      s = s * 6364136223846793005ull + 1442695040888963407ull;
      h[i] = (uint32_t)(s >> 32);
    }
    CHECK(hipMemcpy(in, h.data(), n * 4, hipMemcpyHostToDevice));
  }
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  bool all_ok = true;
  double tile_copy_gbps = 0, pass_gbps = 0;

  auto bench = [&](const char* name, double* gbps_out, auto launch, size_t count = 0) -> int {
    if (count == 0) count = n;  // keys the variant moves
    CHECK(hipMemset(out, 0, n * 4));
    CHECK(hipMemset(sums, 0, 4 * sizeof(unsigned long long)));
    launch();
    hipLaunchKernelGGL(checksum, dim3(2048), dim3(256), 0, 0, (const uint32_t*)in, count, sums);
    hipLaunchKernelGGL(checksum, dim3(2048), dim3(256), 0, 0, (const uint32_t*)out, count, sums + 2);
    unsigned long long hs[4];
    CHECK(hipMemcpy(hs, sums, sizeof(hs), hipMemcpyDeviceToHost));
    const bool ok = hs[0] == hs[2] && hs[1] == hs[3];
    all_ok = all_ok && ok;
    for (int i = 0; i < 3; ++i) launch();
    std::vector<float> ms;
    for (int i = 0; i < 20; ++i) {
      CHECK(hipEventRecord(a, 0));
      launch();
      CHECK(hipEventRecord(b, 0));
      CHECK(hipEventSynchronize(b));
      float t = 0;
      CHECK(hipEventElapsedTime(&t, a, b));
      ms.push_back(t);
    }
    std::sort(ms.begin(), ms.end());
    const double gbps = 8.0 * count / ms[10] / 1e6;
    std::printf("%-34s median %.4f ms  min %.4f ms  %6.0f GB/s  %5.1f %% of 8 TB/s  %s\n", name, ms[10], ms[0], gbps,
                gbps / 80.0, ok ? "permutation ok" : "NOT A PERMUTATION");
    if (gbps_out) *gbps_out = gbps;
    return 0;
  };

#define PATTERN(RUN, label, keep)                                                                                 \
  if (bench(label, keep, [&] {                                                                                    \
        hipLaunchKernelGGL((pass_pattern<RUN>), dim3(tiles), dim3(BLOCK), 0, 0, (const uint32_t*)in, out, tiles, 1u); \
      }))                                                                                                         \
    return 1;

  PATTERN(TILE, "tile copied in place (1 run)", &tile_copy_gbps)
  PATTERN(2304, "8 runs of 2304 keys (9 KiB)", nullptr)
  PATTERN(576, "32 runs of 576 keys", nullptr)
  PATTERN(288, "64 runs of 288 keys", nullptr)
  PATTERN(144, "128 runs of 144 keys (576 bytes)", nullptr)
  PATTERN(72, "256 runs of 72 keys (288 bytes)", &pass_gbps)
  // the same 256 runs with neighbouring tiles on the same XCD, in groups of 8, 64, 512 tiles and an eighth of all tiles
  for (uint32_t group : {8u, 64u, 512u, (tiles + 7) / 8}) {
    char label[64];
    std::snprintf(label, sizeof(label), "256 runs of 72, %u tiles per XCD", group);
    const uint32_t supers = (tiles + 8 * group - 1) / (8 * group);  // whole groups of 8 * group tiles cover all tiles
    if (bench(label, nullptr, [&] {
          hipLaunchKernelGGL((pass_pattern<72, true>), dim3(supers * 8 * group), dim3(BLOCK), 0, 0, (const uint32_t*)in, out,
                             tiles, group);
        }))
      return 1;
  }
  // runs of 64 keys = 256 bytes that start on cache-line boundaries: 16384-key tiles (16 keys per lane), 16382 of them
  // fit the arrays; shorter runs than the pass's 72 keys, but no line is shared between two tiles
  if (bench("256 runs of 64 keys, line-aligned", nullptr, [&] {
        hipLaunchKernelGGL((pass_pattern<64, false, 16>), dim3(16382), dim3(BLOCK), 0, 0, (const uint32_t*)in, out, 16382u, 1u);
      }, (size_t)16382 * 16384))
    return 1;
  PATTERN(36, "512 runs of 36 keys (144 bytes)", nullptr)
  PATTERN(9, "2048 runs of 9 keys (36 bytes)", nullptr)
  // pairs: 2^27 (uint64, uint32) in 16384 tiles of 8192, in buffers of their own; 24 bytes move per pair
  {
    const uint32_t ptiles = 16384;
    const size_t np = (size_t)ptiles * TILE_P;  // 2^27
    uint64_t *kin = nullptr, *kout = nullptr;
    uint32_t *vin = nullptr, *vout = nullptr;
    CHECK(hipMalloc(&kin, np * 8));
    CHECK(hipMalloc(&kout, np * 8));
    CHECK(hipMalloc(&vin, np * 4));
    CHECK(hipMalloc(&vout, np * 4));
    CHECK(hipMemset(kin, 3, np * 8));
    CHECK(hipMemset(vin, 5, np * 4));
    auto pairs = [&](const char* name, auto launch) -> int {
      for (int i = 0; i < 3; ++i) launch();
      std::vector<float> ms;
      for (int i = 0; i < 20; ++i) {
        CHECK(hipEventRecord(a, 0));
        launch();
        CHECK(hipEventRecord(b, 0));
        CHECK(hipEventSynchronize(b));
        float t = 0;
        CHECK(hipEventElapsedTime(&t, a, b));
        ms.push_back(t);
      }
      std::sort(ms.begin(), ms.end());
      const double gbps = 24.0 * np / ms[10] / 1e6;
      std::printf("%-34s median %.4f ms  min %.4f ms  %6.0f GB/s  %5.1f %% of 8 TB/s\n", name, ms[10], ms[0], gbps, gbps / 80.0);
      return 0;
    };
#define PAIRS(RUN, label)                                                                                            \
  if (pairs(label, [&] {                                                                                             \
        hipLaunchKernelGGL((pass_pattern_pairs<RUN>), dim3(ptiles), dim3(BLOCK), 0, 0, (const uint64_t*)kin, kout,   \
                           (const uint32_t*)vin, vout, ptiles);                                                      \
      }))                                                                                                            \
    return 1;
    PAIRS(TILE_P, "pairs: tile copied in place")
    PAIRS(128, "pairs: 64 runs of 128")
    PAIRS(64, "pairs: 128 runs of 64")
    PAIRS(32, "pairs: 256 runs of 32 (a pass)")
    CHECK(hipFree(kin));
    CHECK(hipFree(kout));
    CHECK(hipFree(vin));
    CHECK(hipFree(vout));
  }
  std::printf("a pass's pattern (256 runs of 72 keys) moves %.0f GB/s = %.1f %% of 8 TB/s, %.0f %% of the same tiles copied in place\n",
              pass_gbps, pass_gbps / 80.0, 100.0 * pass_gbps / tile_copy_gbps);
  const bool sane = all_ok && tile_copy_gbps > 2000.0 && pass_gbps > 1000.0;
  std::printf(sane ? "PASSED\n" : "FAILED\n");
  return sane ? 0 : 1;
}
