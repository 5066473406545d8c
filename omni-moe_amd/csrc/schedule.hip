// Expert-centric schedule for gfx950: a stable counting sort of the (token, expert) pairs.
//
// Replaces get_scheduling_info's tail part (omni_moe/ops/triton/omni_scheduler.py:48-101),
// which runs ~12 torch launches including a radix sort and reads two results back to
// the host (:82, :90).  Here the pairs are sorted by expert id with one counting pass when
// N <= 4096 (one bin per expert), two passes (low then high half of the id bits) above that.
// A pass is: per-block bin counts in LDS -> exclusive scan over [bin][block] -> scatter.  The
// scatter is order preserving without any global atomic: a block owns a contiguous tile of
// the input, each of its 4 waves a contiguous quarter; per-wave bin bases come from an LDS
// table, and inside a wave 64 consecutive items rank themselves with ballots.  So a segment
// lists its pairs by ascending pair id, and the result is bit-identical from run to run.
// Offsets are dense over all N experts (an unused expert has an empty segment), so no
// compaction pass is needed, and nothing returns to the host.
#include "common.h"
#include "omni_moe_hip.h"

namespace omni {

constexpr int kScanBlock = 256;
constexpr int kScanPerThread = 16;
constexpr int kScanTile = kScanBlock * kScanPerThread;   // 4096 entries per block
constexpr int kMaxScanBlocks = 1024;                      // <= 4 Mi entries per scan

constexpr int kSortThreads = 256;
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kMaxBins = 4097;                            // 4096 experts (or id slices) + 1 bin for ids outside [0, N)

struct SortPass {
  const int32_t* keys_in;   // expert ids, in the order left by the previous pass
  const int32_t* vals_in;   // pair ids travelling with them; NULL = position (first pass)
  int32_t* keys_out;
  int32_t* vals_out;
  int32_t* tok_out;         // NULL, or pair id / top_k (last pass)
  int32_t* hist;            // [bins][blocks]: counts, then (after the scan) output bases
  int64_t num_pairs;
  int tile;                 // pairs per block, a multiple of 256
  int blocks, bins, bits;   // bits = ceil(log2(bins))
  int shift;                // digit = id >> shift ...
  uint32_t mask;            //   ... & mask (0xFFFFFFFF on the last pass)
  int last;                 // last pass: ids outside [0, N) go to bin bins-1; earlier passes: to bin 0
  uint32_t num_experts;
  int top_k;
};

__device__ __forceinline__ int sort_digit(const SortPass& a, int32_t key) {
  const bool valid = (uint32_t)key < a.num_experts;
  const int d = (int)(((uint32_t)key >> a.shift) & a.mask);
  return valid ? d : (a.last ? a.bins - 1 : 0);
}

__global__ __launch_bounds__(kSortThreads) void sort_count_kernel(const SortPass a) {
  extern __shared__ int32_t cnt[];
  for (int d = threadIdx.x; d < a.bins; d += kSortThreads) cnt[d] = 0;
  __syncthreads();
  const int64_t t0 = (int64_t)blockIdx.x * a.tile;
  const int64_t t1 = t0 + a.tile < a.num_pairs ? t0 + a.tile : a.num_pairs;
  for (int64_t i = t0 + threadIdx.x; i < t1; i += kSortThreads) atomicAdd(&cnt[sort_digit(a, a.keys_in[i])], 1);
  __syncthreads();
  for (int d = threadIdx.x; d < a.bins; d += kSortThreads) a.hist[(int64_t)d * a.blocks + blockIdx.x] = cnt[d];
}

__global__ __launch_bounds__(kSortThreads) void sort_scatter_kernel(const SortPass a) {
  extern __shared__ int32_t tbl[];                       // [waves][bins]: counts, then running output positions
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  for (int d = threadIdx.x; d < a.bins * kSortWaves; d += kSortThreads) tbl[d] = 0;
  __syncthreads();
  const int64_t t0 = (int64_t)blockIdx.x * a.tile;
  const int64_t t1 = t0 + a.tile < a.num_pairs ? t0 + a.tile : a.num_pairs;
  const int64_t w0 = t0 + (int64_t)wave * (a.tile / kSortWaves);                  // this wave's quarter, in order
  const int64_t w1 = w0 + a.tile / kSortWaves < t1 ? w0 + a.tile / kSortWaves : t1;
  int32_t* mine = tbl + wave * a.bins;
  for (int64_t i = w0 + lane; i < w1; i += kWave) atomicAdd(&mine[sort_digit(a, a.keys_in[i])], 1);
  __syncthreads();
  // bases: the block's base of a bin, then wave by wave.  The strided global reads of a thread's
  // bins are all issued before any is used.
  constexpr int kBinsPerThread = (kMaxBins + kSortThreads - 1) / kSortThreads;
  int32_t block_base[kBinsPerThread];
#pragma unroll
  for (int j = 0; j < kBinsPerThread; ++j) {
    const int d = threadIdx.x + j * kSortThreads;
    block_base[j] = d < a.bins ? a.hist[(int64_t)d * a.blocks + blockIdx.x] : 0;
  }
#pragma unroll
  for (int j = 0; j < kBinsPerThread; ++j) {
    const int d = threadIdx.x + j * kSortThreads;
    if (d < a.bins) {
      int32_t base = block_base[j];
#pragma unroll
      for (int w = 0; w < kSortWaves; ++w) {
        const int32_t c = tbl[w * a.bins + d];
        tbl[w * a.bins + d] = base;
        base += c;
      }
    }
  }
  __syncthreads();
  const uint64_t below = (1ull << lane) - 1ull;
  constexpr int kGroup = 8;                                  // steps whose loads are issued together
  for (int64_t g0 = w0; g0 < w1; g0 += kGroup * kWave) {
    int32_t keys[kGroup], vals[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const int64_t i = g0 + u * kWave + lane;
      keys[u] = i < w1 ? a.keys_in[i] : 0;
      vals[u] = i < w1 ? (a.vals_in ? a.vals_in[i] : (int32_t)i) : 0;
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {                       // 64 consecutive items at a time, in order
      const int64_t i = g0 + u * kWave + lane;
      const bool active = i < w1;
      const int32_t key = keys[u], val = vals[u];
      const int d = active ? sort_digit(a, key) : 0;
      uint64_t same = __ballot(active);                      // lanes holding the same bin as this one
      for (int b = 0; b < a.bits; ++b) {
        const bool bit = (d >> b) & 1;
        const uint64_t vote = __ballot(bit && active);
        same &= bit ? vote : ~vote;
      }
      const int rank = __popcll(same & below);
      if (active) {
        const int32_t pos = mine[d] + rank;
        a.keys_out[pos] = key;
        a.vals_out[pos] = val;
        if (a.tok_out) a.tok_out[pos] = val / a.top_k;
        if (rank == 0) mine[d] += __popcll(same);          // one lane per bin; LDS ops of a wave execute in order
      }
    }
  }
}

// offsets[e] = first position whose (sorted) id is >= e; ids outside [0, N) count as N.
__global__ __launch_bounds__(256) void segment_offsets_kernel(const int32_t* __restrict__ sorted_keys, int32_t* __restrict__ offsets,
                                                              int64_t num_pairs, uint32_t num_experts) {
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i <= num_pairs; i += gridDim.x * 256ll) {
    const uint32_t n = num_experts;
    int64_t prev = -1, cur = n;
    if (i > 0) { const uint32_t k = (uint32_t)sorted_keys[i - 1]; prev = k < n ? k : n; }
    if (i < num_pairs) { const uint32_t k = (uint32_t)sorted_keys[i]; cur = k < n ? k : n; }
    for (int64_t e = prev + 1; e <= cur; ++e) offsets[e] = (int32_t)i;
  }
}

// Phase 1: every block scans its tile of 4096 bins locally (exclusive), leaves the
// tile total in tile_sums[block].
__global__ __launch_bounds__(kScanBlock) void scan_tiles_kernel(const int32_t* counts, int32_t* offsets,   // may alias: a thread reads its entries before it writes them
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
      if (cursor) cursor[base + i] = o;
    }
  if ((int)blockIdx.x == num_tiles - 1 && threadIdx.x == 0) offsets[n] = prior + tile_sums[num_tiles - 1];
}

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

static inline int ceil_log2(uint64_t v) { int b = 0; while ((1ull << b) < v) ++b; return b; }

// How the sort of P pairs with ids below N is split into passes and tiles.
struct SortPlan {
  int passes, lo_bits, bins[2], tile, blocks;
  size_t hist_entries;
};
static bool make_plan(int64_t P, int64_t N, SortPlan* pl) {
  const int kb = ceil_log2((uint64_t)N);
  if (kb <= 12) { pl->passes = 1; pl->lo_bits = 0; pl->bins[0] = (int)N + 1; pl->bins[1] = 0; }
  else {
    pl->passes = 2; pl->lo_bits = kb / 2;
    pl->bins[0] = 1 << pl->lo_bits;
    pl->bins[1] = (int)((N + (1ll << pl->lo_bits) - 1) >> pl->lo_bits) + 1;
  }
  const int maxb = pl->bins[0] > pl->bins[1] ? pl->bins[0] : pl->bins[1];
  if (maxb > kMaxBins) return false;                       // N > 16 Mi experts
  int tile = 2048;
  while ((int64_t)maxb * ((P + tile - 1) / tile) > (int64_t)kMaxScanBlocks * kScanTile && tile < (1 << 20)) tile *= 2;
  if ((int64_t)maxb * ((P + tile - 1) / tile) > (int64_t)kMaxScanBlocks * kScanTile) return false;
  pl->tile = tile;
  pl->blocks = (int)((P + tile - 1) / tile);
  if (pl->blocks < 1) pl->blocks = 1;
  pl->hist_entries = (size_t)maxb * pl->blocks;
  return true;
}

}  // namespace omni

// workspace: hist [maxbins*blocks + 1] | scan tile sums [1024] | keys A [P] | keys B [P] | pair ids [P]
extern "C" OMNI_API size_t omni_schedule_workspace_bytes(int64_t num_tokens, int32_t num_experts_per_token, int64_t num_experts) {
  using namespace omni;
  const int64_t P = num_tokens * (int64_t)num_experts_per_token;
  SortPlan pl;
  if (num_tokens < 0 || num_experts_per_token < 0 || num_experts <= 0 || !make_plan(P, num_experts, &pl)) return 0;
  return align_up((pl.hist_entries + 1) * 4, 256) + align_up((size_t)kMaxScanBlocks * 4, 256) + 3 * align_up((size_t)P * 4 + 4, 256);
}

extern "C" OMNI_API int32_t omni_schedule(const int32_t* indices, int32_t* offsets, int32_t* sorted_pair_ids,
                                          int32_t* sorted_token_ids, int64_t num_tokens, int32_t num_experts_per_token,
                                          int64_t num_experts, void* workspace, void* stream) {
  using namespace omni;
  const int64_t N = num_experts, P = num_tokens * (int64_t)num_experts_per_token;
  if (num_tokens < 0 || num_experts_per_token < 0 || N <= 0 || P > INT32_MAX / 2 || N > INT32_MAX / 2) return OMNI_ERR_SHAPE;
  SortPlan pl;
  if (!make_plan(P, N, &pl)) return OMNI_ERR_UNSUPPORTED;
  if (!offsets || (P > 0 && (!indices || !sorted_pair_ids))) return OMNI_ERR_NULL;
  if (!workspace) return OMNI_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  char* w = (char*)workspace;
  int32_t* hist = (int32_t*)w;       w += align_up((pl.hist_entries + 1) * 4, 256);
  int32_t* tile_sums = (int32_t*)w;  w += align_up((size_t)kMaxScanBlocks * 4, 256);
  int32_t* keys_a = (int32_t*)w;     w += align_up((size_t)P * 4 + 4, 256);
  int32_t* keys_b = (int32_t*)w;     w += align_up((size_t)P * 4 + 4, 256);
  int32_t* vals_a = (int32_t*)w;

  const int32_t* sorted_keys = indices;                     // P == 0: nothing to sort
  if (P > 0) {
    for (int pass = 0; pass < pl.passes; ++pass) {
      const bool last = pass == pl.passes - 1;
      SortPass a;
      a.keys_in = pass == 0 ? indices : keys_a;
      a.vals_in = pass == 0 ? nullptr : vals_a;
      a.keys_out = last ? keys_b : keys_a;
      a.vals_out = last ? sorted_pair_ids : vals_a;
      a.tok_out = last ? sorted_token_ids : nullptr;
      a.hist = hist;
      a.num_pairs = P;
      a.tile = pl.tile;
      a.blocks = pl.blocks;
      a.bins = pl.bins[pass];
      a.bits = ceil_log2((uint64_t)a.bins);
      a.shift = pass == 0 ? 0 : pl.lo_bits;
      a.mask = (pl.passes == 2 && pass == 0) ? (uint32_t)((1 << pl.lo_bits) - 1) : 0xFFFFFFFFu;
      a.last = last ? 1 : 0;
      a.num_experts = (uint32_t)N;
      a.top_k = num_experts_per_token;
      const int64_t entries = (int64_t)a.bins * a.blocks;
      const int scan_tiles = (int)((entries + kScanTile - 1) / kScanTile);
      static std::atomic<uint64_t> configured{0};          // tables of up to 4 x 4097 counters exceed the 64 KiB default
      if (hipError_t e = ensure_dynamic_lds((const void*)sort_scatter_kernel, kMaxBins * kSortWaves * 4, configured); e != hipSuccess)
        return OMNI_ERR_HIP_BASE + (int)e;
      hipLaunchKernelGGL(sort_count_kernel, dim3(a.blocks), dim3(kSortThreads), (size_t)a.bins * 4, s, a);
      hipLaunchKernelGGL(scan_tiles_kernel, dim3(scan_tiles), dim3(kScanBlock), 0, s, hist, hist, tile_sums, entries);
      hipLaunchKernelGGL(scan_fixup_kernel, dim3(scan_tiles), dim3(kScanBlock), 0, s, hist, (int32_t*)nullptr, tile_sums, entries, scan_tiles);
      hipLaunchKernelGGL(sort_scatter_kernel, dim3(a.blocks), dim3(kSortThreads), (size_t)a.bins * kSortWaves * 4, s, a);
    }
    sorted_keys = keys_b;
  }
  const unsigned nb = (unsigned)((P + 256) / 256 < 2048 ? (P + 256) / 256 : 2048);
  hipLaunchKernelGGL(segment_offsets_kernel, dim3(nb), dim3(256), 0, s, sorted_keys, offsets, P, (uint32_t)N);
  hipError_t err = hipGetLastError();
  return err == hipSuccess ? OMNI_OK : OMNI_ERR_HIP_BASE + (int)err;
}

// ---- the same schedule for callers that cannot allocate ---------------------------------------
// Code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc have no
// way to bring a workspace.  For them the sort's workspace is a fixed array in device memory that
// each GPU holds from the moment the library is loaded until the process ends.  In host code the
// array's name is only a handle: its device address is looked up once per device with
// hipGetSymbolAddress and kept; every kernel receives that address as its workspace argument.
namespace omni {

static __device__ __align__(256) unsigned char scratch[OMNI_SCHEDULE_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_addr[kMaxDevices];

// Device address of `scratch` on the current device (resolved on the first call per device).
static int scratch_address(void** out) {
  int dev = -1;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return OMNI_ERR_HIP_BASE + (int)e;
  if (dev < 0 || dev >= kMaxDevices) return OMNI_ERR_UNSUPPORTED;
  void* p = g_scratch_addr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)); e != hipSuccess) return OMNI_ERR_HIP_BASE + (int)e;
    if (!p) return OMNI_ERR_SCRATCH;
    g_scratch_addr[dev].store(p, std::memory_order_release);   // concurrent first calls store the same address
  }
  *out = p;
  return OMNI_OK;
}

}  // namespace omni

extern "C" OMNI_API int32_t omni_schedule_noalloc(const int32_t* indices, int32_t* offsets, int32_t* sorted_pair_ids,
                                                  int32_t* sorted_token_ids, int64_t num_tokens, int32_t num_experts_per_token,
                                                  int64_t num_experts, void* stream) {
  using namespace omni;
  const int64_t N = num_experts, P = num_tokens * (int64_t)num_experts_per_token;
  if (num_tokens < 0 || num_experts_per_token < 0 || N <= 0 || P > INT32_MAX / 2 || N > INT32_MAX / 2) return OMNI_ERR_SHAPE;
  SortPlan pl;
  if (!make_plan(P, N, &pl)) return OMNI_ERR_UNSUPPORTED;
  const size_t need = omni_schedule_workspace_bytes(num_tokens, num_experts_per_token, num_experts);
  if (need == 0 || need > (size_t)OMNI_SCHEDULE_NOALLOC_SCRATCH_BYTES) return OMNI_ERR_SCRATCH;
  void* ws = nullptr;
  if (int e = scratch_address(&ws)) return e;
  // every kernel of the sort writes the part of the workspace it later reads (counts, tile sums,
  // keys, pair ids), so nothing of an earlier call's contents has to be cleared
  return omni_schedule(indices, offsets, sorted_pair_ids, sorted_token_ids, num_tokens, num_experts_per_token, num_experts, ws, stream);
}
