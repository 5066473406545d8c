/* A plain C caller that runs one compute entry of libomni_moe_hip.so on the GPU: omni_router_select on device buffers
 * it allocates and fills through the HIP runtime's C API, checked against a scalar loop over the same inputs.
 * Built (gcc) and run by tests/test_gpu_c_client.py on the GPU box. */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "omni_moe_hip.h"

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %d at line %d\n", (int)e_, __LINE__); return 10; } } while (0)

enum { T = 37, R = 8, K = 6 };

int main(void) {
  /* fp32 logits with distinct values, so that ties play no part */
  static float lx[T * R], ly[T * R];
  uint32_t s = 12345u;
  for (int i = 0; i < T * R; ++i) {
    s = s * 1664525u + 1013904223u; lx[i] = -(float)(s >> 8) / 16777216.0f - 0.001f * (float)(i % R);
    s = s * 1664525u + 1013904223u; ly[i] = -(float)(s >> 8) / 16777216.0f - 0.0013f * (float)(i % R);
  }
  void *dlx, *dly, *dscores, *dids;
  CHECK(hipMalloc(&dlx, sizeof lx)); CHECK(hipMalloc(&dly, sizeof ly));
  CHECK(hipMalloc(&dscores, T * K * sizeof(float))); CHECK(hipMalloc(&dids, T * K * sizeof(int32_t)));
  CHECK(hipMemcpy(dlx, lx, sizeof lx, hipMemcpyHostToDevice)); CHECK(hipMemcpy(dly, ly, sizeof ly, hipMemcpyHostToDevice));
  const int32_t code = omni_router_select(dlx, dly, dscores, (int32_t*)dids, T, R, K, OMNI_F32, NULL);
  if (code != OMNI_OK) { printf("omni_router_select: %s\n", omni_error_string(code)); return 11; }
  CHECK(hipDeviceSynchronize());
  static float scores[T * K];
  static int32_t ids[T * K];
  CHECK(hipMemcpy(scores, dscores, sizeof scores, hipMemcpyDeviceToHost)); CHECK(hipMemcpy(ids, dids, sizeof ids, hipMemcpyDeviceToHost));
  /* brute force: the K largest of the R*R sums per token, by repeated maximum */
  for (int t = 0; t < T; ++t) {
    char taken[R * R] = {0};
    for (int j = 0; j < K; ++j) {
      int best = -1; float bs = 0.f;
      for (int e = 0; e < R * R; ++e) {
        if (taken[e]) continue;
        const float v = lx[t * R + e / R] + ly[t * R + e % R];
        if (best < 0 || v > bs) { best = e; bs = v; }
      }
      taken[best] = 1;
      if (ids[t * K + j] != best || scores[t * K + j] != bs) {
        printf("token %d slot %d: got id %d score %.9g, want id %d score %.9g\n", t, j, ids[t * K + j], scores[t * K + j], best, bs);
        return 12;
      }
    }
  }
  CHECK(hipFree(dlx)); CHECK(hipFree(dly)); CHECK(hipFree(dscores)); CHECK(hipFree(dids));
  printf("c abi gpu ok: %d tokens routed\n", T);
  return 0;
}
