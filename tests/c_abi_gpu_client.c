/* A plain C caller that runs compute entries of libomni_moe_hip.so on the GPU: omni_router_select on device buffers
 * it allocates and fills through the HIP runtime's C API, checked against a scalar loop over the same inputs; then
 * omni_init(), and straight after it -- no eager call came before -- HIP-graph captures of
 *   - omni_linear_fwd at a shape whose kernel needs 128 KiB of dynamic LDS: without omni_init() the call would have
 *     to raise that kernel's limit with hipFuncSetAttribute inside the capture; omni_init() has done it for every kernel,
 *   - omni_schedule and omni_schedule_noalloc side by side (the second on the device scratch that omni_init() resolved),
 * each replayed three times and checked against scalar loops.
 * Built (gcc) and run by tests/test_gpu_c_client.py on the GPU box. */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "omni_moe_hip.h"

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %d at line %d\n", (int)e_, __LINE__); return 10; } } while (0)

enum { T = 37, R = 8, K = 6 };
enum { ST = 300, SK = 4, SN = 4096, SP = ST * SK };

enum { GM = 2048, GN = 2048, GK = 64 };

/* bf16 bits of a small integer (exactly representable) and back */
static uint16_t bf16_of_int(int v) { float f = (float)v; uint32_t u; memcpy(&u, &f, 4); return (uint16_t)(u >> 16); }
static float float_of_bf16(uint16_t b) { uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }

/* omni_linear_fwd inside a stream capture, straight after omni_init().  2048 x 2048 outputs make the library pick its
 * 128 x 128 tile, whose kernel needs 128 KiB of dynamic LDS.  Operands are small integers, so every product and sum is
 * exact and the result must equal the scalar loop bit for bit. */
static int captured_gemm(void) {
  uint16_t* x = (uint16_t*)malloc((size_t)GM * GK * 2); uint16_t* w = (uint16_t*)malloc((size_t)GN * GK * 2);
  uint16_t* y = (uint16_t*)malloc((size_t)GM * GN * 2);
  int8_t* xi = (int8_t*)malloc((size_t)GM * GK); int8_t* wi = (int8_t*)malloc((size_t)GN * GK);
  if (!x || !w || !y || !xi || !wi) return 30;
  uint32_t s = 4242u;
  for (int i = 0; i < GM * GK; ++i) { s = s * 1664525u + 1013904223u; xi[i] = (int8_t)((int)((s >> 12) % 5) - 2); x[i] = bf16_of_int(xi[i]); }
  for (int i = 0; i < GN * GK; ++i) { s = s * 1664525u + 1013904223u; wi[i] = (int8_t)((int)((s >> 12) % 3) - 1); w[i] = bf16_of_int(wi[i]); }
  void *dx, *dw, *dy;
  CHECK(hipMalloc(&dx, (size_t)GM * GK * 2)); CHECK(hipMalloc(&dw, (size_t)GN * GK * 2)); CHECK(hipMalloc(&dy, (size_t)GM * GN * 2));
  CHECK(hipMemcpy(dx, x, (size_t)GM * GK * 2, hipMemcpyHostToDevice)); CHECK(hipMemcpy(dw, w, (size_t)GN * GK * 2, hipMemcpyHostToDevice));
  hipStream_t stream; hipGraph_t graph; hipGraphExec_t exec;
  CHECK(hipStreamCreate(&stream));
  CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
  const int32_t code = omni_linear_fwd(dx, dw, NULL, dy, GM, GK, GN, OMNI_BF16, stream);
  const hipError_t end = hipStreamEndCapture(stream, &graph);
  if (code != OMNI_OK) { printf("omni_linear_fwd under capture: %s\n", omni_error_string(code)); return 31; }
  CHECK(end);
  CHECK(hipGraphInstantiate(&exec, graph, NULL, NULL, 0));
  for (int rep = 0; rep < 3; ++rep) {
    CHECK(hipMemset(dy, 0xff, (size_t)GM * GN * 2));
    CHECK(hipGraphLaunch(exec, stream));
    CHECK(hipStreamSynchronize(stream));
    CHECK(hipMemcpy(y, dy, (size_t)GM * GN * 2, hipMemcpyDeviceToHost));
    for (int m = 0; m < GM; ++m)
      for (int n = 0; n < GN; ++n) {
        int acc = 0;
        for (int k = 0; k < GK; ++k) acc += xi[m * GK + k] * wi[n * GK + k];      /* |acc| <= 128: exact in bf16 */
        if (float_of_bf16(y[(size_t)m * GN + n]) != (float)acc) { printf("gemm replay %d: y[%d][%d] = %g, want %d\n", rep, m, n, float_of_bf16(y[(size_t)m * GN + n]), acc); return 32; }
      }
  }
  CHECK(hipGraphExecDestroy(exec)); CHECK(hipGraphDestroy(graph)); CHECK(hipStreamDestroy(stream));
  CHECK(hipFree(dx)); CHECK(hipFree(dw)); CHECK(hipFree(dy));
  free(x); free(w); free(y); free(xi); free(wi);
  return 0;
}

/* omni_schedule and omni_schedule_noalloc inside one stream capture: no eager call of this shape came before */
static int captured_schedule(void) {
  static int32_t ids[SP], offsets[SN + 1], pairs[SP], tokens[SP], want_off[SN + 1], fill[SN];
  uint32_t s = 777u;
  for (int i = 0; i < SP; ++i) { s = s * 1664525u + 1013904223u; ids[i] = (int32_t)((s >> 10) % SN); }
  const size_t ws_bytes = omni_schedule_workspace_bytes(ST, SK, SN);
  void *dids, *doff[2], *dpairs[2], *dtok[2], *dws;
  CHECK(hipMalloc(&dids, sizeof ids)); CHECK(hipMalloc(&dws, ws_bytes));
  for (int v = 0; v < 2; ++v) { CHECK(hipMalloc(&doff[v], sizeof offsets)); CHECK(hipMalloc(&dpairs[v], sizeof pairs)); CHECK(hipMalloc(&dtok[v], sizeof tokens)); }
  CHECK(hipMemcpy(dids, ids, sizeof ids, hipMemcpyHostToDevice));
  hipStream_t stream; hipGraph_t graph; hipGraphExec_t exec;
  CHECK(hipStreamCreate(&stream));
  CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
  const int32_t code = omni_schedule((const int32_t*)dids, (int32_t*)doff[0], (int32_t*)dpairs[0], (int32_t*)dtok[0], ST, SK, SN, dws, stream);
  const int32_t code2 = omni_schedule_noalloc((const int32_t*)dids, (int32_t*)doff[1], (int32_t*)dpairs[1], (int32_t*)dtok[1], ST, SK, SN, stream);
  const hipError_t end = hipStreamEndCapture(stream, &graph);
  if (code != OMNI_OK) { printf("omni_schedule under capture: %s\n", omni_error_string(code)); return 22; }
  if (code2 != OMNI_OK) { printf("omni_schedule_noalloc under capture: %s\n", omni_error_string(code2)); return 25; }
  CHECK(end);
  CHECK(hipGraphInstantiate(&exec, graph, NULL, NULL, 0));
  for (int i = 0; i <= SN; ++i) want_off[i] = 0;
  for (int i = 0; i < SP; ++i) want_off[ids[i] + 1]++;
  for (int i = 0; i < SN; ++i) want_off[i + 1] += want_off[i];
  for (int rep = 0; rep < 3; ++rep) {
    for (int v = 0; v < 2; ++v) { CHECK(hipMemset(doff[v], 0xff, sizeof offsets)); CHECK(hipMemset(dpairs[v], 0xff, sizeof pairs)); CHECK(hipMemset(dtok[v], 0xff, sizeof tokens)); }
    CHECK(hipGraphLaunch(exec, stream));
    CHECK(hipStreamSynchronize(stream));
    for (int v = 0; v < 2; ++v) {
      CHECK(hipMemcpy(offsets, doff[v], sizeof offsets, hipMemcpyDeviceToHost)); CHECK(hipMemcpy(pairs, dpairs[v], sizeof pairs, hipMemcpyDeviceToHost));
      CHECK(hipMemcpy(tokens, dtok[v], sizeof tokens, hipMemcpyDeviceToHost));
      for (int i = 0; i < SN; ++i) fill[i] = 0;
      for (int i = 0; i <= SN; ++i) if (offsets[i] != want_off[i]) { printf("replay %d entry %d: offsets[%d] = %d, want %d\n", rep, v, i, offsets[i], want_off[i]); return 23; }
      for (int i = 0; i < SP; ++i) {                       /* stable: pair i lands at its expert's next free slot */
        const int32_t slot = want_off[ids[i]] + fill[ids[i]]++;
        if (pairs[slot] != i || tokens[slot] != i / SK) { printf("replay %d entry %d: slot %d holds pair %d token %d, want %d %d\n", rep, v, slot, pairs[slot], tokens[slot], i, i / SK); return 24; }
      }
    }
  }
  CHECK(hipGraphExecDestroy(exec)); CHECK(hipGraphDestroy(graph)); CHECK(hipStreamDestroy(stream));
  CHECK(hipFree(dids)); CHECK(hipFree(dws));
  for (int v = 0; v < 2; ++v) { CHECK(hipFree(doff[v])); CHECK(hipFree(dpairs[v])); CHECK(hipFree(dtok[v])); }
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
  int32_t init = omni_init();
  if (init != OMNI_OK) { printf("omni_init: %s\n", omni_error_string(init)); return 20; }
  if (omni_init() != OMNI_OK) { printf("second omni_init failed\n"); return 21; }
  const int gemm = captured_gemm();
  if (gemm) return gemm;
  const int sched = captured_schedule();
  if (sched) return sched;
  printf("c abi gpu ok: %d tokens routed, a %d x %d x %d product and %d pairs scheduled (with and without workspace) from captured graphs\n", T, GM, GN, GK, SP);
  return 0;
}
