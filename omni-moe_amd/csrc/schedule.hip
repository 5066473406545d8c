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
//            its own tile for its share), scans the totals over the bins, and has its output
//            bases; block 0 writes them out as the segment offsets.  Then it places its pairs.
// Scattered 4-byte stores are bound by the requests one CU can issue, so up to 8 scatter blocks share
// a tile: each places one part of it and counts the parts before its own itself.
// The scatter is order preserving without any global atomic: each of the block's 8 waves owns a
// contiguous eighth of the part; per-wave bin bases come from an LDS table, and inside a wave 64
// consecutive items rank themselves (an LDS add per item, ballots where two items of a step meet
// in a bin).  So a segment lists its pairs by ascending pair id, and the result is bit-identical
// from run to run.  Offsets are dense over all N experts (an unused expert has an empty segment),
// so no compaction pass is needed, and nothing returns to the host.  Few, large tiles (32 where the
// 16-bit counters allow) keep the histogram small: every scatter block reads it once, one batch of loads.
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
constexpr int kRowBatch = 32;                             // histogram rows whose loads are in flight together
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
  int sub;                  // scatter blocks per tile (a power of two that divides tile / 8)
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
  constexpr int kBatch = 8;                              // loads in flight per thread
  for (int64_t i0 = t0 + threadIdx.x; i0 < t1; i0 += kBatch * kSortThreads) {
    int32_t key[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int64_t i = i0 + u * kSortThreads;
      key[u] = i < t1 ? a.keys_in[i] : 0;
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
      if (i0 + u * kSortThreads < t1) atomicAdd(&cnt[sort_digit(a, key[u])], 1);
  }
  __syncthreads();
  for (int d = threadIdx.x; d < a.stride; d += kSortThreads) a.hist[(int64_t)blockIdx.x * a.stride + d] = (uint16_t)cnt[d];
}

__global__ __launch_bounds__(kSortThreads) void sort_scatter_kernel(const SortPass a) {
  extern __shared__ int32_t tbl[];                       // [waves][stride]: counts, then running output positions; then [stride] bin bases
  __shared__ int32_t wave_tot[kSortWaves];
  int32_t* bin_base = tbl + kSortWaves * a.stride;
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  // The histogram rows come from other blocks' writes, i.e. from memory: thread t takes bins 8t .. 8t+7 of every row
  // (one 16-byte load per row), kRowBatch rows in flight together, the first batch while the tile is being counted.
  const int d0 = threadIdx.x * kBinChunk;
  const bool active = d0 < a.stride && d0 < kSortThreads * kBinChunk;
  auto load_rows = [&](u32x4_t (&row)[kRowBatch], int first) {
#pragma unroll
    for (int j = 0; j < kRowBatch; ++j)
      row[j] = (active && first + j < a.blocks) ? *(const u32x4_t*)(a.hist + (int64_t)(first + j) * a.stride + d0) : u32x4_t{0, 0, 0, 0};
  };
  u32x4_t early[kRowBatch];
  load_rows(early, 0);
  for (int d = threadIdx.x * 4; d < a.stride * (kSortWaves + 1); d += kSortThreads * 4) *(u32x4_t*)(tbl + d) = u32x4_t{0, 0, 0, 0};   // stride % 8 == 0
  __syncthreads();
  // a.sub blocks share a tile (the scattered stores are bound by the requests one CU can issue, so they are spread
  // over many CUs); block sb of a tile places the sb-th part of it, after the parts before it
  const int tile_idx = (int)blockIdx.x / a.sub, sb = (int)blockIdx.x % a.sub;
  const int64_t t0 = (int64_t)tile_idx * a.tile;
  const int64_t t1 = t0 + a.tile < a.num_pairs ? t0 + a.tile : a.num_pairs;
  const int share = a.tile / a.sub, per_wave = share / kSortWaves;
  const int64_t s0 = t0 + (int64_t)sb * share < t1 ? t0 + (int64_t)sb * share : t1;             // earlier parts of the tile: [t0, s0)
  const int64_t w0 = s0 + (int64_t)wave * per_wave < t1 ? s0 + (int64_t)wave * per_wave : t1;   // this wave's eighth of the part, in order
  const int64_t w1 = w0 + per_wave < t1 ? w0 + per_wave : t1;
  int32_t* mine = tbl + wave * a.stride;
  constexpr int kGroup = 8;                              // steps of 64 items whose loads are issued together
  for (int64_t i0 = t0 + threadIdx.x; i0 < s0; i0 += kGroup * kSortThreads) {   // what the tile's earlier parts put into each bin
    int32_t key[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const int64_t i = i0 + u * kSortThreads;
      key[u] = i < s0 ? a.keys_in[i] : 0;
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u)
      if (i0 + u * kSortThreads < s0) atomicAdd(&bin_base[sort_digit(a, key[u])], 1);
  }
  for (int64_t g0 = w0; g0 < w1; g0 += kGroup * kWave) {
    int32_t key[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const int64_t i = g0 + u * kWave + lane;
      key[u] = i < w1 ? a.keys_in[i] : 0;
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u)
      if (g0 + u * kWave + lane < w1) atomicAdd(&mine[sort_digit(a, key[u])], 1);
  }
  __syncthreads();

  // Output bases.  The rows above this block's give what earlier tiles put into each bin, all rows the bin's total.
  // An exclusive scan of the totals over the bins (thread order = bin order) gives each bin's first position.
  // 512 threads cover 4096 bins; the one bin beyond them (ids outside the table, when there are 4096 experts) is
  // summed by wave 0, a row per lane.
  int32_t before[kBinChunk], rest[kBinChunk];
#pragma unroll
  for (int i = 0; i < kBinChunk; ++i) before[i] = rest[i] = 0;
  auto add_rows = [&](const u32x4_t (&row)[kRowBatch], int first) {
    auto add = [&](int32_t (&acc)[kBinChunk], const u32x4_t& r) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[2 * i] += (int32_t)(r[i] & 0xffffu);
        acc[2 * i + 1] += (int32_t)(r[i] >> 16);
      }
    };
#pragma unroll
    for (int j = 0; j < kRowBatch; ++j) {
      if (first + j < tile_idx) add(before, row[j]);      // a scalar branch: the row index is uniform
      else add(rest, row[j]);
    }
  };
  add_rows(early, 0);
  for (int b0 = kRowBatch; b0 < a.blocks; b0 += kRowBatch) {
    u32x4_t row[kRowBatch];
    load_rows(row, b0);
    add_rows(row, b0);
  }
  const int tail_bin = kSortThreads * kBinChunk;         // 4096
  int32_t tail_before = 0, tail_total = 0;
  if (a.bins > tail_bin && wave == 0) {
    for (int b = lane; b < a.blocks; b += kWave) {
      const int32_t c = a.hist[(int64_t)b * a.stride + tail_bin];
      tail_total += c;
      tail_before += b < tile_idx ? c : 0;
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
        bin_base[d] += excl + before[i];                   // on top of the earlier parts' count
      }
      excl += before[i] + rest[i];
    }
    if (a.bins > tail_bin && threadIdx.x == 0) {         // the bin behind all others starts where they end
      if (a.offsets_out && blockIdx.x == 0) a.offsets_out[tail_bin] = all;
      bin_base[tail_bin] += all + tail_before;
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

  // Placement, 64 consecutive items at a time and in order.  Position = the bin's running base + the number of earlier
  // lanes of the step with the same bin.  Every lane reads the base, then bumps it; a lane that finds the base already
  // bumped shares its bin with another lane of its step, and only then are the lanes of that bin ranked by lane number
  // (whatever order the adds took effect in).  LDS executes a wave's instructions in order, so the reads and adds of all
  // steps of a group are issued back to back (a later step sees the earlier steps' adds) and waited for once.
  const uint64_t below = (1ull << lane) - 1ull;
  for (int64_t g0 = w0; g0 < w1; g0 += kGroup * kWave) {
    int32_t keys[kGroup], vals[kGroup], dig[kGroup], pos[kGroup], bumped[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const int64_t i = g0 + u * kWave + lane;
      keys[u] = i < w1 ? a.keys_in[i] : 0;
      vals[u] = i < w1 ? (a.vals_in ? a.vals_in[i] : (int32_t)i) : 0;
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const bool active = g0 + u * kWave + lane < w1;
      dig[u] = active ? sort_digit(a, keys[u]) : 0;
      pos[u] = bumped[u] = 0;
      if (active) {
        pos[u] = mine[dig[u]];
        bumped[u] = atomicAdd(&mine[dig[u]], 1);
      }
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const bool active = g0 + u * kWave + lane < w1;
      const int d = dig[u];
      uint64_t shared = __ballot(active && bumped[u] != pos[u]);   // the non-first lanes of shared bins
      while (shared) {
        const int l = __builtin_ctzll(shared);
        const int v = __shfl(d, l, kWave);
        const uint64_t grp = __ballot(active && d == v);           // all lanes of that bin; they read the same base
        if (active && d == v) pos[u] += __popcll(grp & below);
        shared &= ~grp;
      }
      if (active) {
        if (a.keys_out) a.keys_out[pos[u]] = keys[u];
        a.vals_out[pos[u]] = vals[u];
        if (a.tok_out) a.tok_out[pos[u]] = (int32_t)(((uint64_t)(uint32_t)vals[u] * a.inv_top_k) >> 40);   // val / top_k
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
  int passes, lo_bits, bins[2], stride, tile, blocks, sub;
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
  // every scatter block sums the whole histogram, one 16-byte load per row and thread: 32 rows (tiles) are one batch of
  // loads; more only where a tile would outgrow its 16-bit counters
  constexpr int want = 32;
  int64_t tile = (P + want - 1) / want;
  tile = (tile + 1023) / 1024 * 1024;
  if (tile < 1024) tile = 1024;
  if (tile > kMaxTile) tile = kMaxTile;
  if ((P + tile - 1) / tile > kMaxSortBlocks) return false;   // more than 64 Mi pairs
  pl->tile = (int)tile;
  pl->blocks = (int)((P + tile - 1) / tile);
  if (pl->blocks < 1) pl->blocks = 1;
  pl->hist_entries = (size_t)pl->stride * pl->blocks;
  // scatter blocks per tile: towards one block per CU, each part at least 8 waves x 64 items (tile is a multiple of 1024)
  pl->sub = 1;
  while (pl->sub < 8 && pl->blocks * pl->sub * 2 <= 256 && pl->tile / (pl->sub * 2) >= 512) pl->sub *= 2;
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
      a.sub = pl.sub;
      a.bins = pl.bins[pass];
      a.stride = pl.stride;
      a.bits = ceil_log2((uint64_t)a.bins);
      a.shift = pass == 0 ? 0 : pl.lo_bits;
      a.mask = (pl.passes == 2 && pass == 0) ? (uint32_t)((1 << pl.lo_bits) - 1) : 0xFFFFFFFFu;
      a.last = last ? 1 : 0;
      a.num_experts = (uint32_t)N;
      a.inv_top_k = num_experts_per_token > 0 ? ((1ull << 40) + num_experts_per_token - 1) / (uint64_t)num_experts_per_token : 0;
      hipLaunchKernelGGL(sort_count_kernel, dim3(a.blocks), dim3(kSortThreads), (size_t)a.stride * 4, s, a);
      hipLaunchKernelGGL(sort_scatter_kernel, dim3(a.blocks * a.sub), dim3(kSortThreads), (size_t)a.stride * (kSortWaves + 1) * 4, s, a);
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
