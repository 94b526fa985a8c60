// What the memory system of the GPU gives to kernels that do nothing but move bytes: plain
// read, write and copy kernels over 1 GiB, in the tile shapes the library's kernels use.
// Every bandwidth-bound kernel of the library is measured against 8 TB/s (the published HBM
// peak); these kernels show how much of that peak any kernel can reach on the machine at
// hand, so that "fraction of peak" can also be read as "fraction of what a copy reaches".
// Standalone HIP program (does not use the library); prints one line per kernel and PASSED
// when the numbers are sane.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <vector>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define CHECK(expr)                                                                  \
  do {                                                                               \
    hipError_t e_ = (expr);                                                          \
    if (e_ != hipSuccess) {                                                          \
      std::printf("%s failed: %s\n", #expr, hipGetErrorString(e_));                  \
      return 1;                                                                      \
    }                                                                                \
  } while (0)

// BLOCK threads move U 16-byte vectors each; a workgroup's tile is BLOCK * U * 16 bytes.
template <int BLOCK, int U>
__global__ __launch_bounds__(BLOCK) void ceiling_copy(const u32x4* __restrict__ in, u32x4* __restrict__ out) {
  const size_t base = (size_t)blockIdx.x * BLOCK * U + threadIdx.x;
  u32x4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) v[u] = in[base + (size_t)u * BLOCK];
#pragma unroll
  for (int u = 0; u < U; ++u) out[base + (size_t)u * BLOCK] = v[u];
}

template <int BLOCK, int U>
__global__ __launch_bounds__(BLOCK) void ceiling_read(const u32x4* __restrict__ in, u32x4* __restrict__ out) {
  const size_t base = (size_t)blockIdx.x * BLOCK * U + threadIdx.x;
  u32x4 v[U];
  u32x4 a = {0, 0, 0, 0};
#pragma unroll
  for (int u = 0; u < U; ++u) v[u] = in[base + (size_t)u * BLOCK];
#pragma unroll
  for (int u = 0; u < U; ++u) a += v[u];
  if (a.x == 0x12345678u) out[0] = a;  // never true for the input used: keeps the loads alive
}

template <int BLOCK, int U>
__global__ __launch_bounds__(BLOCK) void ceiling_write(u32x4* __restrict__ out) {
  const size_t base = (size_t)blockIdx.x * BLOCK * U + threadIdx.x;
  const u32x4 a = {1, 2, 3, 4};
#pragma unroll
  for (int u = 0; u < U; ++u) out[base + (size_t)u * BLOCK] = a;
}

int main() {
  const size_t n = (size_t)1 << 28;  // 4-byte elements: 1 GiB per array
  const size_t vectors = n / 4;
  int *in = nullptr, *out = nullptr;
  CHECK(hipMalloc(&in, n * 4));
  CHECK(hipMalloc(&out, n * 4));
  CHECK(hipMemset(in, 1, n * 4));
  CHECK(hipMemset(out, 1, n * 4));
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  double best_copy = 0, best_read = 0, best_write = 0;

  auto bench = [&](const char* name, double bytes, double& best, auto launch) -> int {
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
    const double gbps = bytes / ms[10] / 1e6;
    std::printf("%-28s median %.4f ms  min %.4f ms  %7.0f GB/s  %5.1f %% of 8 TB/s\n", name, ms[10], ms[0], gbps,
                gbps / 80.0);
    best = std::max(best, gbps);
    return 0;
  };

#define COPY(B, U)                                                                                         \
  if (bench("copy  " #B " threads x " #U, 8.0 * n, best_copy, [&] {                                        \
        hipLaunchKernelGGL((ceiling_copy<B, U>), dim3(vectors / B / U), dim3(B), 0, 0, (const u32x4*)in,   \
                           (u32x4*)out);                                                                   \
      }))                                                                                                  \
    return 1;
#define READ(B, U)                                                                                         \
  if (bench("read  " #B " threads x " #U, 4.0 * n, best_read, [&] {                                        \
        hipLaunchKernelGGL((ceiling_read<B, U>), dim3(vectors / B / U), dim3(B), 0, 0, (const u32x4*)in,   \
                           (u32x4*)out);                                                                   \
      }))                                                                                                  \
    return 1;
#define WRITE(B, U)                                                                                        \
  if (bench("write " #B " threads x " #U, 4.0 * n, best_write, [&] {                                       \
        hipLaunchKernelGGL((ceiling_write<B, U>), dim3(vectors / B / U), dim3(B), 0, 0, (u32x4*)out);      \
      }))                                                                                                  \
    return 1;

  COPY(256, 1) COPY(256, 2) COPY(256, 4) COPY(512, 2) COPY(1024, 2) COPY(1024, 4)
  COPY(1024, 12)  // the scan kernel's tile: 1024 threads x 12 vectors = 192 KiB
  READ(256, 2) READ(256, 4) READ(256, 8) READ(1024, 8)  // 1024 x 8: the reduce kernel's tile
  WRITE(256, 2) WRITE(256, 4) WRITE(1024, 4)
  std::printf("best copy %.0f GB/s (%.1f %%), best read %.0f GB/s (%.1f %%), best write %.0f GB/s (%.1f %%)\n", best_copy,
              best_copy / 80.0, best_read, best_read / 80.0, best_write, best_write / 80.0);
  // sanity only: a machine whose copy stays under a quarter of the peak is not the one the
  // library's figures were taken on
  const bool sane = best_copy > 2000.0 && best_read > 2000.0 && best_write > 2000.0;
  std::printf(sane ? "PASSED\n" : "FAILED\n");
  return sane ? 0 : 1;
}
