// Expert-centric schedule for gfx950: a counting sort of the (token, expert) pairs.
//
// Replaces get_scheduling_info's tail part (omni_moe/ops/triton/omni_scheduler.py:48-101),
// which runs ~12 torch launches including a radix sort and reads two results back to
// the host (:82, :90).  Here: histogram over the N expert bins -> exclusive prefix sum ->
// scatter, five short launches, nothing returns to the host.  Offsets are dense over all
// N experts (an unused expert has an empty segment), so no compaction pass is needed.
#include "common.h"
#include "omni_moe_hip.h"

namespace omni {

constexpr int kScanBlock = 256;
constexpr int kScanPerThread = 16;
constexpr int kScanTile = kScanBlock * kScanPerThread;   // 4096 bins per block
constexpr int kMaxScanBlocks = 1024;                      // N <= 4 Mi experts

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += gridDim.x * 256ll) p[i] = v;
}

// Ids outside [0, N) are dropped here and in the scatter (they get no slot), so a bad
// id can never write out of bounds.
__global__ __launch_bounds__(256) void pair_histogram_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ counts,
                                                             int64_t num_pairs, uint32_t num_experts) {
  for (int64_t p = blockIdx.x * 256ll + threadIdx.x; p < num_pairs; p += gridDim.x * 256ll) {
    const uint32_t e = (uint32_t)ids[p];
    if (e < num_experts) atomicAdd(&counts[e], 1);
  }
}

// Phase 1: every block scans its tile of 4096 bins locally (exclusive), leaves the
// tile total in tile_sums[block].
__global__ __launch_bounds__(kScanBlock) void scan_tiles_kernel(const int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                                int32_t* __restrict__ tile_sums, int64_t n) {
  __shared__ int32_t wave_tot[kScanBlock / kWave];
  const int64_t base = (int64_t)blockIdx.x * kScanTile + threadIdx.x * kScanPerThread;
  int32_t v[kScanPerThread], sum = 0;
#pragma unroll
  for (int i = 0; i < kScanPerThread; ++i) {
    v[i] = (base + i < n) ? counts[base + i] : 0;
    sum += v[i];
  }
  // inclusive scan of the per-thread sums across the wave
  int32_t inc = sum;
  const int lane = lane_id(), wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int32_t o = __shfl_up(inc, d, kWave);
    if (lane >= d) inc += o;
  }
  if (lane == kWave - 1) wave_tot[wave] = inc;
  __syncthreads();
  int32_t before = inc - sum;
  for (int w = 0; w < wave; ++w) before += wave_tot[w];
#pragma unroll
  for (int i = 0; i < kScanPerThread; ++i) {
    if (base + i < n) offsets[base + i] = before;
    before += v[i];
  }
  if (threadIdx.x == kScanBlock - 1) tile_sums[blockIdx.x] = before;
}

// Phase 2: add the sum of the preceding tiles; also seed the scatter cursors and
// write offsets[n] = total.
__global__ __launch_bounds__(kScanBlock) void scan_fixup_kernel(int32_t* __restrict__ offsets, int32_t* __restrict__ cursor,
                                                                const int32_t* __restrict__ tile_sums, int64_t n, int num_tiles) {
  __shared__ int32_t wave_tot[kScanBlock / kWave];
  int32_t part = 0;
  for (int i = threadIdx.x; i < (int)blockIdx.x; i += kScanBlock) part += tile_sums[i];
  int32_t w = part;
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) w += __shfl_xor(w, m, kWave);
  if (lane_id() == 0) wave_tot[threadIdx.x >> 6] = w;
  __syncthreads();
  int32_t prior = 0;
#pragma unroll
  for (int i = 0; i < kScanBlock / kWave; ++i) prior += wave_tot[i];
  const int64_t base = (int64_t)blockIdx.x * kScanTile + threadIdx.x * kScanPerThread;
#pragma unroll
  for (int i = 0; i < kScanPerThread; ++i)
    if (base + i < n) {
      const int32_t o = offsets[base + i] + prior;
      offsets[base + i] = o;
      cursor[base + i] = o;
    }
  if ((int)blockIdx.x == num_tiles - 1 && threadIdx.x == 0) offsets[n] = prior + tile_sums[num_tiles - 1];
}

__global__ __launch_bounds__(256) void pair_scatter_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ cursor,
                                                           int32_t* __restrict__ sorted_pair_ids, int32_t* __restrict__ sorted_token_ids,
                                                           int64_t num_pairs, int top_k, uint32_t num_experts) {
  for (int64_t p = blockIdx.x * 256ll + threadIdx.x; p < num_pairs; p += gridDim.x * 256ll) {
    const uint32_t e = (uint32_t)ids[p];
    if (e >= num_experts) continue;
    const int32_t pos = atomicAdd(&cursor[e], 1);
    sorted_pair_ids[pos] = (int32_t)p;
    if (sorted_token_ids) sorted_token_ids[pos] = (int32_t)(p / top_k);
  }
}

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace omni

extern "C" OMNI_API size_t omni_schedule_workspace_bytes(int64_t num_tokens, int32_t num_experts_per_token, int64_t num_experts) {
  (void)num_tokens; (void)num_experts_per_token;
  if (num_experts < 0) return 0;
  // cursors [N] + tile sums
  return omni::align_up((size_t)num_experts * 4, 256) + (size_t)omni::kMaxScanBlocks * 4;
}

extern "C" OMNI_API int32_t omni_schedule(const int32_t* indices, int32_t* offsets, int32_t* sorted_pair_ids,
                                 int32_t* sorted_token_ids, int64_t num_tokens, int32_t num_experts_per_token,
                                 int64_t num_experts, void* workspace, void* stream) {
  using namespace omni;
  const int64_t N = num_experts, P = num_tokens * (int64_t)num_experts_per_token;
  if (num_tokens < 0 || num_experts_per_token < 0 || N <= 0 || P > INT32_MAX) return OMNI_ERR_SHAPE;
  const int num_tiles = (int)((N + kScanTile - 1) / kScanTile);
  if (num_tiles > kMaxScanBlocks) return OMNI_ERR_UNSUPPORTED;
  if (!offsets || (P > 0 && (!indices || !sorted_pair_ids))) return OMNI_ERR_NULL;
  if (!workspace) return OMNI_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  int32_t* cursor = (int32_t*)workspace;
  int32_t* tile_sums = (int32_t*)((char*)workspace + align_up((size_t)N * 4, 256));

  const unsigned nb_n = (unsigned)((N + 255) / 256 < 2048 ? (N + 255) / 256 : 2048);
  const unsigned nb_p = (unsigned)((P + 255) / 256 < 4096 ? (P + 255) / 256 : 4096);
  hipLaunchKernelGGL(fill_i32_kernel, dim3(nb_n), dim3(256), 0, s, cursor, N, 0);
  if (P > 0) hipLaunchKernelGGL(pair_histogram_kernel, dim3(nb_p), dim3(256), 0, s, indices, cursor, P, (uint32_t)N);
  hipLaunchKernelGGL(scan_tiles_kernel, dim3(num_tiles), dim3(kScanBlock), 0, s, cursor, offsets, tile_sums, N);
  hipLaunchKernelGGL(scan_fixup_kernel, dim3(num_tiles), dim3(kScanBlock), 0, s, offsets, cursor, tile_sums, N, num_tiles);
  if (P > 0)
    hipLaunchKernelGGL(pair_scatter_kernel, dim3(nb_p), dim3(256), 0, s, indices, cursor, sorted_pair_ids, sorted_token_ids,
                       P, (int)num_experts_per_token, (uint32_t)N);
  hipError_t err = hipGetLastError();
  return err == hipSuccess ? OMNI_OK : OMNI_ERR_HIP_BASE + (int)err;
}
