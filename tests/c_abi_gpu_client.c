/* A plain C caller that runs one compute entry of libomni_moe_hip.so on the GPU: omni_router_select on device buffers
 * it allocates and fills through the HIP runtime's C API, checked against a scalar loop over the same inputs; then
 * omni_init() followed by a HIP-graph capture of omni_schedule for a shape that never ran eagerly (its kernel needs
 * more than the default dynamic LDS, which omni_init has already arranged), replayed and checked the same way.
 * Built (gcc) and run by tests/test_gpu_c_client.py on the GPU box. */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "omni_moe_hip.h"

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %d at line %d\n", (int)e_, __LINE__); return 10; } } while (0)

enum { T = 37, R = 8, K = 6 };
enum { ST = 300, SK = 4, SN = 4096, SP = ST * SK };

/* omni_schedule inside a stream capture, straight after omni_init(): no eager call of this shape came before */
static int captured_schedule(void) {
  static int32_t ids[SP], offsets[SN + 1], pairs[SP], tokens[SP], want_off[SN + 1], fill[SN];
  uint32_t s = 777u;
  for (int i = 0; i < SP; ++i) { s = s * 1664525u + 1013904223u; ids[i] = (int32_t)((s >> 10) % SN); }
  int32_t code = omni_init();
  if (code != OMNI_OK) { printf("omni_init: %s\n", omni_error_string(code)); return 20; }
  if (omni_init() != OMNI_OK) { printf("second omni_init failed\n"); return 21; }
  const size_t ws_bytes = omni_schedule_workspace_bytes(ST, SK, SN);
  void *dids, *doff, *dpairs, *dtok, *dws;
  CHECK(hipMalloc(&dids, sizeof ids)); CHECK(hipMalloc(&doff, sizeof offsets)); CHECK(hipMalloc(&dpairs, sizeof pairs));
  CHECK(hipMalloc(&dtok, sizeof tokens)); CHECK(hipMalloc(&dws, ws_bytes));
  CHECK(hipMemcpy(dids, ids, sizeof ids, hipMemcpyHostToDevice));
  hipStream_t stream; hipGraph_t graph; hipGraphExec_t exec;
  CHECK(hipStreamCreate(&stream));
  CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
  code = omni_schedule((const int32_t*)dids, (int32_t*)doff, (int32_t*)dpairs, (int32_t*)dtok, ST, SK, SN, dws, stream);
  const hipError_t end = hipStreamEndCapture(stream, &graph);
  if (code != OMNI_OK) { printf("omni_schedule under capture: %s\n", omni_error_string(code)); return 22; }
  CHECK(end);
  CHECK(hipGraphInstantiate(&exec, graph, NULL, NULL, 0));
  for (int i = 0; i <= SN; ++i) want_off[i] = 0;
  for (int i = 0; i < SP; ++i) want_off[ids[i] + 1]++;
  for (int i = 0; i < SN; ++i) want_off[i + 1] += want_off[i];
  for (int rep = 0; rep < 3; ++rep) {
    CHECK(hipMemset(doff, 0xff, sizeof offsets)); CHECK(hipMemset(dpairs, 0xff, sizeof pairs)); CHECK(hipMemset(dtok, 0xff, sizeof tokens));
    CHECK(hipGraphLaunch(exec, stream));
    CHECK(hipStreamSynchronize(stream));
    CHECK(hipMemcpy(offsets, doff, sizeof offsets, hipMemcpyDeviceToHost)); CHECK(hipMemcpy(pairs, dpairs, sizeof pairs, hipMemcpyDeviceToHost));
    CHECK(hipMemcpy(tokens, dtok, sizeof tokens, hipMemcpyDeviceToHost));
    for (int i = 0; i < SN; ++i) fill[i] = 0;
    for (int i = 0; i <= SN; ++i) if (offsets[i] != want_off[i]) { printf("replay %d: offsets[%d] = %d, want %d\n", rep, i, offsets[i], want_off[i]); return 23; }
    for (int i = 0; i < SP; ++i) {                       /* stable: pair i lands at its expert's next free slot */
      const int32_t slot = want_off[ids[i]] + fill[ids[i]]++;
      if (pairs[slot] != i || tokens[slot] != i / SK) { printf("replay %d: slot %d holds pair %d token %d, want %d %d\n", rep, slot, pairs[slot], tokens[slot], i, i / SK); return 24; }
    }
  }
  CHECK(hipGraphExecDestroy(exec)); CHECK(hipGraphDestroy(graph)); CHECK(hipStreamDestroy(stream));
  CHECK(hipFree(dids)); CHECK(hipFree(doff)); CHECK(hipFree(dpairs)); CHECK(hipFree(dtok)); CHECK(hipFree(dws));
  return 0;
}

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
  const int sched = captured_schedule();
  if (sched) return sched;
  printf("c abi gpu ok: %d tokens routed, %d pairs scheduled from a captured graph\n", T, SP);
  return 0;
}
