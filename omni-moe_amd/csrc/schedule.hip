// Expert-centric schedule for gfx950: a stable counting sort of the (token, expert) pairs.
//
// Replaces get_scheduling_info's tail part (omni_moe/ops/triton/omni_scheduler.py:48-101),
// which runs ~12 torch launches including a radix sort and reads two results back to
// the host (:82, :90).  Here the pairs are sorted by expert id with one counting pass when
// N <= 4096 (one bin per expert), two passes (low then high half of the id bits) above that.
// A pass is two kernels:
//   count:   every block counts the bins of its contiguous tile of the input in LDS and writes
//            them as one row of hist[block][bin] (coalesced, 16-bit counters: a tile has fewer
//            than 65536 pairs; the histogram is the only scratch);
//   scatter: every block sums the rows of hist (all of them for the bins' totals, the rows above
//            its own for its share), scans the totals over the bins, and has its output bases;
//            block 0 writes them out as the segment offsets.  Then it places its tile.
// The scatter is order preserving without any global atomic: each of the block's 8 waves owns a
// contiguous eighth of the tile; per-wave bin bases come from an LDS table, and inside a wave 64
// consecutive items rank themselves with ballots.  So a segment lists its pairs by ascending pair
// id, and the result is bit-identical from run to run.  Offsets are dense over all N experts (an
// unused expert has an empty segment), so no compaction pass is needed, and nothing returns to
// the host.  Few, large tiles (about 131072 / bins blocks) keep the histogram small: it is read
// once per block.
#include "common.h"
#include "omni_moe_hip.h"

namespace omni {

constexpr int kSortThreads = 512;
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kMaxBins = 4097;                            // 4096 experts (or id slices) + 1 bin for ids outside [0, N)
constexpr int kBinChunk = 8;                              // bins a thread sums at a time (one 16-byte load per histogram row)
constexpr int kMaxStride = (kMaxBins + kBinChunk - 1) / kBinChunk * kBinChunk;
constexpr int kMaxSortBlocks = 1024;
constexpr int kMaxTile = 63 * 1024;                       // counters are 16 bits wide
constexpr int kRowBatch = 16;                             // histogram rows whose loads are in flight together
static_assert(kMaxBins <= kSortThreads * kBinChunk + 1, "the scan covers 8 bins per thread plus one");

struct SortPass {
  const int32_t* keys_in;   // expert ids, in the order left by the previous pass
  const int32_t* vals_in;   // pair ids travelling with them; NULL = position (first pass)
  int32_t* keys_out;        // NULL: not needed (single pass)
  int32_t* vals_out;
  int32_t* tok_out;         // NULL, or pair id / top_k (last pass)
  int32_t* offsets_out;     // NULL, or [bins]: first output position of every bin (single pass: the segment offsets)
  uint16_t* hist;           // [blocks][stride] bin counts of every tile
  int64_t num_pairs;
  int tile;                 // pairs per block, a multiple of 1024
  int blocks, bins, stride, bits;   // stride = bins rounded up to 8; bits = ceil(log2(bins))
  int shift;                // digit = id >> shift ...
  uint32_t mask;            //   ... & mask (0xFFFFFFFF on the last pass)
  int last;                 // last pass: ids outside [0, N) go to bin bins-1; earlier passes: to bin 0
  uint32_t num_experts;
  uint64_t inv_top_k;       // ceil(2^40 / top_k): (v * inv_top_k) >> 40 == v / top_k for every v < 2^31 and top_k <= 2^9
};

__device__ __forceinline__ int sort_digit(const SortPass& a, int32_t key) {
  const bool valid = (uint32_t)key < a.num_experts;
  const int d = (int)(((uint32_t)key >> a.shift) & a.mask);
  return valid ? d : (a.last ? a.bins - 1 : 0);
}

__global__ __launch_bounds__(kSortThreads) void sort_count_kernel(const SortPass a) {
  extern __shared__ int32_t cnt[];
  for (int d = threadIdx.x; d < a.stride; d += kSortThreads) cnt[d] = 0;
  __syncthreads();
  const int64_t t0 = (int64_t)blockIdx.x * a.tile;
  const int64_t t1 = t0 + a.tile < a.num_pairs ? t0 + a.tile : a.num_pairs;
  for (int64_t i = t0 + threadIdx.x; i < t1; i += kSortThreads) atomicAdd(&cnt[sort_digit(a, a.keys_in[i])], 1);
  __syncthreads();
  for (int d = threadIdx.x; d < a.stride; d += kSortThreads) a.hist[(int64_t)blockIdx.x * a.stride + d] = (uint16_t)cnt[d];
}

__global__ __launch_bounds__(kSortThreads) void sort_scatter_kernel(const SortPass a) {
  extern __shared__ int32_t tbl[];                       // [waves][stride]: counts, then running output positions; then [stride] bin bases
  __shared__ int32_t wave_tot[kSortWaves];
  int32_t* bin_base = tbl + kSortWaves * a.stride;
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  for (int d = threadIdx.x * 4; d < a.stride * kSortWaves; d += kSortThreads * 4) *(u32x4_t*)(tbl + d) = u32x4_t{0, 0, 0, 0};   // stride % 8 == 0
  __syncthreads();
  const int64_t t0 = (int64_t)blockIdx.x * a.tile;
  const int64_t t1 = t0 + a.tile < a.num_pairs ? t0 + a.tile : a.num_pairs;
  const int per_wave = a.tile / kSortWaves;
  const int64_t w0 = t0 + (int64_t)wave * per_wave < t1 ? t0 + (int64_t)wave * per_wave : t1;   // this wave's eighth, in order
  const int64_t w1 = w0 + per_wave < t1 ? w0 + per_wave : t1;
  int32_t* mine = tbl + wave * a.stride;
  for (int64_t i = w0 + lane; i < w1; i += kWave) atomicAdd(&mine[sort_digit(a, a.keys_in[i])], 1);
  __syncthreads();

  // Output bases.  Thread t takes bins 8t .. 8t+7 and walks down the histogram rows: the rows above this block's
  // give what earlier tiles put into each bin, all rows the bin's total.  An exclusive scan of the totals over the
  // bins (thread order = bin order) gives each bin's first position.  The rows come from other blocks' writes, i.e.
  // from memory: the loads of kRowBatch rows are in flight together.  512 threads cover 4096 bins; the one bin
  // beyond them (ids outside the table, when there are 4096 experts) is summed by wave 0, a row per lane.
  const int d0 = threadIdx.x * kBinChunk;
  const bool active = d0 < a.stride && d0 < kSortThreads * kBinChunk;
  int32_t before[kBinChunk], rest[kBinChunk];
#pragma unroll
  for (int i = 0; i < kBinChunk; ++i) before[i] = rest[i] = 0;
  auto add_rows = [&](int32_t (&acc)[kBinChunk], int first, int end) {
    for (int b0 = first; b0 < end; b0 += kRowBatch) {
      u32x4_t row[kRowBatch];
#pragma unroll
      for (int j = 0; j < kRowBatch; ++j)
        row[j] = (active && b0 + j < end) ? *(const u32x4_t*)(a.hist + (int64_t)(b0 + j) * a.stride + d0) : u32x4_t{0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < kRowBatch; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t pair = row[j][i];
          acc[2 * i] += (int32_t)(pair & 0xffffu);
          acc[2 * i + 1] += (int32_t)(pair >> 16);
        }
    }
  };
  add_rows(before, 0, (int)blockIdx.x);
  add_rows(rest, (int)blockIdx.x, a.blocks);
  const int tail_bin = kSortThreads * kBinChunk;         // 4096
  int32_t tail_before = 0, tail_total = 0;
  if (a.bins > tail_bin && wave == 0) {
    for (int b = lane; b < a.blocks; b += kWave) {
      const int32_t c = a.hist[(int64_t)b * a.stride + tail_bin];
      tail_total += c;
      tail_before += b < (int)blockIdx.x ? c : 0;
    }
#pragma unroll
    for (int m = kWave / 2; m >= 1; m >>= 1) {
      tail_total += __shfl_xor(tail_total, m, kWave);
      tail_before += __shfl_xor(tail_before, m, kWave);
    }
  }
  {
    int32_t tsum = 0;
#pragma unroll
    for (int i = 0; i < kBinChunk; ++i) tsum += before[i] + rest[i];
    int32_t inc = tsum;                                  // inclusive scan across the wave
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int32_t o = __shfl_up(inc, d, kWave);
      if (lane >= d) inc += o;
    }
    if (lane == kWave - 1) wave_tot[wave] = inc;
    __syncthreads();
    int32_t excl = inc - tsum, all = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
      excl += w < wave ? wave_tot[w] : 0;
      all += wave_tot[w];
    }
#pragma unroll
    for (int i = 0; i < kBinChunk; ++i) {
      const int d = d0 + i;
      if (active && d < a.bins) {
        if (a.offsets_out && blockIdx.x == 0) a.offsets_out[d] = excl;
        bin_base[d] = excl + before[i];
      }
      excl += before[i] + rest[i];
    }
    if (a.bins > tail_bin && threadIdx.x == 0) {         // the bin behind all others starts where they end
      if (a.offsets_out && blockIdx.x == 0) a.offsets_out[tail_bin] = all;
      bin_base[tail_bin] = all + tail_before;
    }
    __syncthreads();
  }
  // per-wave bases: consecutive threads take consecutive bins (no bank conflicts), wave by wave down the table
  for (int d = threadIdx.x; d < a.bins; d += kSortThreads) {
    int32_t base = bin_base[d];
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
      const int32_t c = tbl[w * a.stride + d];
      tbl[w * a.stride + d] = base;
      base += c;
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
      // Position = the bin's running base + the number of earlier lanes of this step with the same bin.  Every lane
      // reads the base, then bumps it; a lane that finds the base already bumped shares its bin with another lane of
      // the step.  Only then are the lanes of that bin ranked by lane number (whatever order the adds took effect in).
      int32_t pos = 0, bumped = 0;
      if (active) {
        pos = mine[d];
        bumped = atomicAdd(&mine[d], 1);
      }
      uint64_t shared = __ballot(active && bumped != pos);   // the non-first lanes of shared bins
      while (shared) {
        const int l = __builtin_ctzll(shared);
        const int v = __shfl(d, l, kWave);
        const uint64_t grp = __ballot(active && d == v);     // all lanes of that bin; they read the same base
        if (active && d == v) pos += __popcll(grp & below);
        shared &= ~grp;
      }
      if (active) {
        if (a.keys_out) a.keys_out[pos] = key;
        a.vals_out[pos] = val;
        if (a.tok_out) a.tok_out[pos] = (int32_t)(((uint64_t)(uint32_t)val * a.inv_top_k) >> 40);   // val / top_k
      }
    }
  }
}

// offsets[e] = first position whose (sorted) id is >= e; ids outside [0, N) count as N.  Two-pass sorts only:
// their last pass has a bin per high half of the id, not per expert.
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

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

static inline int ceil_log2(uint64_t v) { int b = 0; while ((1ull << b) < v) ++b; return b; }

// How the sort of P pairs with ids below N is split into passes and tiles.
struct SortPlan {
  int passes, lo_bits, bins[2], stride, tile, blocks;
  size_t hist_entries;
};
static bool make_plan(int64_t P, int64_t N, SortPlan* pl) {
  const int kb = ceil_log2((uint64_t)N);
  if (N + 1 <= kMaxBins) { pl->passes = 1; pl->lo_bits = 0; pl->bins[0] = (int)N + 1; pl->bins[1] = 0; }
  else {
    pl->passes = 2; pl->lo_bits = kb / 2;
    pl->bins[0] = 1 << pl->lo_bits;
    pl->bins[1] = (int)((N + (1ll << pl->lo_bits) - 1) >> pl->lo_bits) + 1;
  }
  const int maxb = pl->bins[0] > pl->bins[1] ? pl->bins[0] : pl->bins[1];
  if (maxb > kMaxBins) return false;                       // N > 16 Mi experts
  pl->stride = (maxb + kBinChunk - 1) / kBinChunk * kBinChunk;
  // every block reads the whole histogram: about 128 Ki counters of it (32 tiles at 4097 bins, 256 at 512),
  // more where a tile would outgrow its 16-bit counters
  int want = ((1 << 17) + maxb - 1) / maxb;
  want = want < 1 ? 1 : (want > 256 ? 256 : want);
  int64_t tile = (P + want - 1) / want;
  tile = (tile + 1023) / 1024 * 1024;
  if (tile < 1024) tile = 1024;
  if (tile > kMaxTile) tile = kMaxTile;
  if ((P + tile - 1) / tile > kMaxSortBlocks) return false;   // more than 64 Mi pairs
  pl->tile = (int)tile;
  pl->blocks = (int)((P + tile - 1) / tile);
  if (pl->blocks < 1) pl->blocks = 1;
  pl->hist_entries = (size_t)pl->stride * pl->blocks;
  return true;
}

// up to 9 x 4104 counters exceed the 64 KiB default
static LdsKernel g_scatter_lds{(const void*)sort_scatter_kernel, kMaxStride * (kSortWaves + 1) * 4};

}  // namespace omni

// workspace: hist [blocks][stride] | two-pass sorts only: keys A [P] | keys B [P] | pair ids [P]
extern "C" OMNI_API size_t omni_schedule_workspace_bytes(int64_t num_tokens, int32_t num_experts_per_token, int64_t num_experts) {
  using namespace omni;
  const int64_t P = num_tokens * (int64_t)num_experts_per_token;
  SortPlan pl;
  if (num_tokens < 0 || num_experts_per_token < 0 || num_experts <= 0 || !make_plan(P, num_experts, &pl)) return 0;
  return align_up(pl.hist_entries * 2, 256) + (pl.passes == 2 ? 3 * align_up((size_t)P * 4 + 4, 256) : 0);
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
  uint16_t* hist = (uint16_t*)w;     w += align_up(pl.hist_entries * 2, 256);
  int32_t* keys_a = (int32_t*)w;     w += align_up((size_t)P * 4 + 4, 256);      // the three arrays exist for two-pass sorts only
  int32_t* keys_b = (int32_t*)w;     w += align_up((size_t)P * 4 + 4, 256);
  int32_t* vals_a = (int32_t*)w;

  if (hipError_t e = g_scatter_lds.ensure(); e != hipSuccess) return OMNI_ERR_HIP_BASE + (int)e;
  const bool single = pl.passes == 1;
  if (single || P > 0) {
    for (int pass = 0; pass < pl.passes; ++pass) {
      const bool last = pass == pl.passes - 1;
      SortPass a;
      a.keys_in = pass == 0 ? indices : keys_a;
      a.vals_in = pass == 0 ? nullptr : vals_a;
      a.keys_out = single ? nullptr : (last ? keys_b : keys_a);
      a.vals_out = last ? sorted_pair_ids : vals_a;
      a.tok_out = last ? sorted_token_ids : nullptr;
      a.offsets_out = single ? offsets : nullptr;          // one bin per expert: the bins' first positions ARE the offsets
      a.hist = hist;
      a.num_pairs = P;
      a.tile = pl.tile;
      a.blocks = pl.blocks;
      a.bins = pl.bins[pass];
      a.stride = pl.stride;
      a.bits = ceil_log2((uint64_t)a.bins);
      a.shift = pass == 0 ? 0 : pl.lo_bits;
      a.mask = (pl.passes == 2 && pass == 0) ? (uint32_t)((1 << pl.lo_bits) - 1) : 0xFFFFFFFFu;
      a.last = last ? 1 : 0;
      a.num_experts = (uint32_t)N;
      a.inv_top_k = num_experts_per_token > 0 ? ((1ull << 40) + num_experts_per_token - 1) / (uint64_t)num_experts_per_token : 0;
      hipLaunchKernelGGL(sort_count_kernel, dim3(a.blocks), dim3(kSortThreads), (size_t)a.stride * 4, s, a);
      hipLaunchKernelGGL(sort_scatter_kernel, dim3(a.blocks), dim3(kSortThreads), (size_t)a.stride * (kSortWaves + 1) * 4, s, a);
    }
  }
  if (!single) {
    const int32_t* sorted_keys = P > 0 ? keys_b : indices;  // P == 0: nothing was sorted, every offset is 0
    const unsigned nb = (unsigned)((P + 256) / 256 < 2048 ? (P + 256) / 256 : 2048);
    hipLaunchKernelGGL(segment_offsets_kernel, dim3(nb), dim3(256), 0, s, sorted_keys, offsets, P, (uint32_t)N);
  }
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

int schedule_scratch_prepare() {
  void* p = nullptr;
  return scratch_address(&p);
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
