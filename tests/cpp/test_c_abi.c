/* The C ABI from plain C: reduce of 1..n through malloc / memcpy / two-phase temp storage. */
#include <stdio.h>
#include <stdlib.h>
#include <thrust_amd.h>

#define CHECK(x) do { int rc_ = (x); if (rc_) { printf("FAIL %s -> %d (%s)\n", #x, rc_, thrust_amd_error_string(rc_)); return 1; } } while (0)

int main(void) {
  const uint64_t n = 100003;
  int32_t* h = (int32_t*)malloc(n * sizeof(int32_t));
  for (uint64_t i = 0; i < n; i++) h[i] = (int32_t)(i + 1);
  void *d = NULL, *temp = NULL, *d_out = NULL;
  CHECK(thrust_amd_malloc(&d, n * sizeof(int32_t)));
  CHECK(thrust_amd_malloc(&d_out, sizeof(int32_t)));
  CHECK(thrust_amd_memcpy(d, h, n * sizeof(int32_t), THRUST_AMD_H2D, NULL));
  size_t bytes = 0;
  int32_t init = 7, out = 0;
  CHECK(thrust_amd_reduce(NULL, &bytes, d, n, THRUST_AMD_I32, THRUST_AMD_PLUS, &init, d_out, NULL));
  CHECK(thrust_amd_malloc(&temp, bytes));
  CHECK(thrust_amd_reduce(temp, &bytes, d, n, THRUST_AMD_I32, THRUST_AMD_PLUS, &init, d_out, NULL));
  CHECK(thrust_amd_memcpy(&out, d_out, sizeof out, THRUST_AMD_D2H, NULL));
  const int64_t expect = (int64_t)n * (int64_t)(n + 1) / 2 + 7;
  /* status codes for misuse, no abort */
  size_t small = 1;
  int rc = thrust_amd_reduce(temp, &small, d, n, THRUST_AMD_I32, THRUST_AMD_PLUS, &init, d_out, NULL);
  int rc2 = thrust_amd_reduce(NULL, &bytes, d, n, 99, THRUST_AMD_PLUS, &init, d_out, NULL);
  CHECK(thrust_amd_free(temp));
  CHECK(thrust_amd_free(d));
  CHECK(thrust_amd_free(d_out));
  free(h);
  if ((int32_t)expect != out || rc == 0 || rc2 == 0) { printf("FAIL result %d expect %d rc %d rc2 %d\n", out, (int32_t)expect, rc, rc2); return 1; }
  printf("PASS c_abi reduce = %d, version %d\n", out, thrust_amd_version());
  return 0;
}
