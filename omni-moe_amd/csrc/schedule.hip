// Expert-centric schedule for gfx950: a stable counting sort of the (token, expert) pairs.
//
// Replaces get_scheduling_info's tail part (omni_moe/ops/triton/omni_scheduler.py:48-101),
// which runs ~12 torch launches including a radix sort and reads two results back to
// the host (:82, :90).  Here the pairs are sorted by expert id with one counting pass when
// N <= 4096 (one bin per expert), two passes (low then high half of the id bits) above that.
// A pass is two kernels:
//   count:   every block counts the bins of its contiguous tile of the input in LDS and writes
//            them as one row of hist[tile][bin] (16-bit counters: a tile has fewer than 65536
//            pairs), plus the row's sum over each of the 8 bin slices;
//   scatter: the bins are cut into 8 slices and a block places the pairs of ONE tile that fall
//            into ONE slice.  It sums its slice of the hist rows (all rows for the bins' totals,
//            the rows above its tile for its share), the slice sums of the slices below it, scans
//            the totals, and has its output bases; the blocks of tile 0 write them out as the
//            segment offsets.
// Why slices: the scattered 4-byte stores are what the pass costs.  Slice s belongs to the blocks
// with blockIdx % 8 == s, which the dispatcher places on XCD s, so every output line is written
// through ONE L2 (which merges the stores of a line before it goes to memory) and the stores are
// spread over all CUs; and a block's tables cover an eighth of the bins, so zeroing, summing,
// scanning them is an eighth of the work.  The price is that a tile's keys are read by 8 blocks.
// The scatter is order preserving without any global atomic: each of the block's 8 waves owns a
// contiguous eighth of the tile; per-wave bin bases come from an LDS table, and inside a wave 64
// consecutive items rank themselves (an LDS add per item, ballots where two items of a step meet
// in a bin).  So a segment lists its pairs by ascending pair id, and the result is bit-identical
// from run to run.  Offsets are dense over all N experts (an unused expert has an empty segment),
// so no compaction pass is needed, and nothing returns to the host.
#include "common.h"
#include "omni_moe_hip.h"

namespace omni {

constexpr int kSortThreads = 512;
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kSlices = 8;                                // bin slices = XCDs
constexpr int kMaxBins = 4097;                            // 4096 experts (or id slices) + 1 bin for ids outside [0, N)
constexpr int kBinChunk = 8;                              // bins per 16-byte load of a histogram row
constexpr int kMaxWidth = ((kMaxBins + kSlices - 1) / kSlices + kBinChunk - 1) / kBinChunk * kBinChunk;   // bins per slice: 520
constexpr int kMaxSortTiles = 1024;
constexpr int kMaxTile = 63 * 1024;                       // counters are 16 bits wide
constexpr int kRowBatch = 8;                              // histogram rows a thread has in flight
constexpr int kGroup = 8;                                 // steps of 64 items whose loads are issued together
static_assert(kSlices == kSortWaves, "the count kernel sums slice w in wave w");

struct SortPass {
  const int32_t* keys_in;   // expert ids, in the order left by the previous pass
  const int32_t* vals_in;   // pair ids travelling with them; NULL = position (first pass)
  int32_t* keys_out;        // NULL: not needed (single pass)
  int32_t* vals_out;
  int32_t* tok_out;         // NULL, or pair id / top_k (last pass)
  int32_t* offsets_out;     // NULL, or [bins]: first output position of every bin (single pass: the segment offsets)
  uint16_t* hist;           // [tiles][stride] bin counts of every tile
  uint32_t* slice_tot;      // [tiles][8] the same counts summed over each slice
  int64_t num_pairs;
  int tile;                 // pairs per tile, a multiple of 1024
  int tiles, bins;
  int width, stride;        // bins per slice (a multiple of 8); stride = 8 * width >= bins
  int shift;                // digit = id >> shift ...
  uint32_t mask;            //   ... & mask (0xFFFFFFFF on the last pass)
  int last;                 // last pass: ids outside [0, N) go to bin bins-1; earlier passes: to bin 0
  uint32_t num_experts;
  uint64_t inv_top_k;       // ceil(2^s / top_k) with s = inv_shift = 30 + ceil(log2(top_k)): (v * inv_top_k) >> s == v / top_k for
  int inv_shift;            // every pair id v < 2^30 (the excess v * (inv_top_k * top_k - 2^s) / (top_k * 2^s) stays below
                            // 1 / top_k, and the product below 2^62)
};

__device__ __forceinline__ int sort_digit(const SortPass& a, int32_t key) {
  const bool valid = (uint32_t)key < a.num_experts;
  const int d = (int)(((uint32_t)key >> a.shift) & a.mask);
  return valid ? d : (a.last ? a.bins - 1 : 0);
}

__device__ __forceinline__ int32_t wave_sum_i32(int32_t v) {
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}

__global__ __launch_bounds__(kSortThreads) void sort_count_kernel(const SortPass a) {
  extern __shared__ int32_t cnt[];                       // [stride]
  for (int d = threadIdx.x; d < a.stride; d += kSortThreads) cnt[d] = 0;
  __syncthreads();
  const int64_t t0 = (int64_t)blockIdx.x * a.tile;
  const int64_t t1 = t0 + a.tile < a.num_pairs ? t0 + a.tile : a.num_pairs;
  for (int64_t i0 = t0 + threadIdx.x; i0 < t1; i0 += kGroup * kSortThreads) {
    int32_t key[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const int64_t i = i0 + u * kSortThreads;
      key[u] = i < t1 ? a.keys_in[i] : 0;
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u)
      if (i0 + u * kSortThreads < t1) atomicAdd(&cnt[sort_digit(a, key[u])], 1);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < a.stride / kBinChunk; c += kSortThreads) {    // 8 counters per 16-byte store
    const int32_t* v = cnt + c * kBinChunk;
    *(u32x4_t*)(a.hist + (int64_t)blockIdx.x * a.stride + c * kBinChunk) =
        u32x4_t{(uint32_t)v[0] | ((uint32_t)v[1] << 16), (uint32_t)v[2] | ((uint32_t)v[3] << 16),
                (uint32_t)v[4] | ((uint32_t)v[5] << 16), (uint32_t)v[6] | ((uint32_t)v[7] << 16)};
  }
  const int lane = lane_id(), wave = threadIdx.x >> 6;   // wave w sums slice w
  int32_t sum = 0;
  for (int d = lane; d < a.width; d += kWave) sum += cnt[wave * a.width + d];
  sum = wave_sum_i32(sum);
  if (lane == 0) a.slice_tot[(int64_t)blockIdx.x * kSlices + wave] = (uint32_t)sum;
}

__global__ __launch_bounds__(kSortThreads) void sort_scatter_kernel(const SortPass a) {
  __shared__ int32_t tbl[kSortWaves][kMaxWidth];         // per wave and bin: count, then running output position
  __shared__ int32_t bin_base[kMaxWidth], before_s[kMaxWidth], total_s[kMaxWidth];
  __shared__ int32_t below_s;                            // pairs in the slices below this one, all tiles
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  const int tile_idx = (int)blockIdx.x / kSlices, slice = (int)blockIdx.x % kSlices;
  const int lo = slice * a.width;                        // this block's bins: lo .. lo + width - 1
  // The histogram rows come from other blocks' writes, i.e. from memory.  Thread t sums chunk t % C (8 bins, one
  // 16-byte load per row) of the rows t / C, t / C + G, ..; the first batch of loads flies while the tile is counted.
  const int C = a.width / kBinChunk, G = kSortThreads / C;
  const int chunk = threadIdx.x % C, group = threadIdx.x / C;
  const bool summing = group < G;
  auto load_rows = [&](u32x4_t (&row)[kRowBatch], int first) {
#pragma unroll
    for (int j = 0; j < kRowBatch; ++j) {
      const int r = first + j * G;
      row[j] = (summing && r < a.tiles) ? *(const u32x4_t*)(a.hist + (int64_t)r * a.stride + lo + chunk * kBinChunk) : u32x4_t{0, 0, 0, 0};
    }
  };
  u32x4_t early[kRowBatch];
  load_rows(early, group);
  for (int d = threadIdx.x; d < kSortWaves * kMaxWidth; d += kSortThreads) (&tbl[0][0])[d] = 0;
  for (int d = threadIdx.x; d < a.width; d += kSortThreads) bin_base[d] = before_s[d] = total_s[d] = 0;
  if (threadIdx.x == 0) below_s = 0;
  __syncthreads();

  const int64_t t0 = (int64_t)tile_idx * a.tile;
  const int64_t t1 = t0 + a.tile < a.num_pairs ? t0 + a.tile : a.num_pairs;
  const int per_wave = a.tile / kSortWaves;
  const int64_t w0 = t0 + (int64_t)wave * per_wave < t1 ? t0 + (int64_t)wave * per_wave : t1;   // this wave's eighth, in order
  const int64_t w1 = w0 + per_wave < t1 ? w0 + per_wave : t1;
  int32_t* mine = tbl[wave];
  for (int64_t g0 = w0; g0 < w1; g0 += kGroup * kWave) {
    int32_t key[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const int64_t i = g0 + u * kWave + lane;
      key[u] = i < w1 ? a.keys_in[i] : 0;
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const int d = sort_digit(a, key[u]) - lo;
      if (g0 + u * kWave + lane < w1 && (uint32_t)d < (uint32_t)a.width) atomicAdd(&mine[d], 1);
    }
  }

  // what the slices below this one hold, over all tiles
  {
    int32_t part = 0;
    for (int e = threadIdx.x; e < a.tiles * kSlices; e += kSortThreads)
      part += (e % kSlices) < slice ? (int32_t)a.slice_tot[e] : 0;
    part = wave_sum_i32(part);
    if (lane == 0 && part) atomicAdd(&below_s, part);
  }
  // this slice of the histogram rows: what earlier tiles put into each bin, and each bin's total
  {
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
        if (first + j * G < tile_idx) add(before, row[j]);
        else add(rest, row[j]);                            // rows past the last tile were loaded as zeros
      }
    };
    add_rows(early, group);
    for (int r0 = group + kRowBatch * G; r0 < a.tiles; r0 += kRowBatch * G) {
      u32x4_t row[kRowBatch];
      load_rows(row, r0);
      add_rows(row, r0);
    }
    if (summing) {
#pragma unroll
      for (int i = 0; i < kBinChunk; ++i) {
        if (before[i]) atomicAdd(&before_s[chunk * kBinChunk + i], before[i]);
        if (before[i] + rest[i]) atomicAdd(&total_s[chunk * kBinChunk + i], before[i] + rest[i]);
      }
    }
  }
  __syncthreads();

  // exclusive scan of the slice's totals (wave 0, a run of consecutive bins per lane): every bin's first position
  if (wave == 0) {
    const int per = (a.width + kWave - 1) / kWave, b0 = lane * per;
    int32_t sum = 0;
    for (int i = 0; i < per; ++i) sum += b0 + i < a.width ? total_s[b0 + i] : 0;
    int32_t inc = sum;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int32_t o = __shfl_up(inc, d, kWave);
      if (lane >= d) inc += o;
    }
    int32_t excl = below_s + inc - sum;
    for (int i = 0; i < per; ++i) {
      const int b = b0 + i;
      if (b < a.width) {
        if (a.offsets_out && tile_idx == 0 && lo + b < a.bins) a.offsets_out[lo + b] = excl;
        bin_base[b] = excl + before_s[b];
        excl += total_s[b];
      }
    }
  }
  __syncthreads();
  // per-wave bases: consecutive threads take consecutive bins (no bank conflicts), wave by wave down the table
  for (int d = threadIdx.x; d < a.width; d += kSortThreads) {
    int32_t base = bin_base[d];
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
      const int32_t c = tbl[w][d];
      tbl[w][d] = base;
      base += c;
    }
  }
  __syncthreads();

  // Placement, 64 consecutive items at a time and in order; only the items of this block's slice take part.
  // Position = the bin's running base + the number of earlier lanes of the step with the same bin.  Every lane
  // reads the base, then bumps it; a lane that finds the base already bumped shares its bin with another lane of
  // its step, and only then are the lanes of that bin ranked by lane number (whatever order the adds took effect
  // in).  LDS executes a wave's instructions in order, so the reads and adds of all steps of a group are issued
  // back to back (a later step sees the earlier steps' adds) and waited for once.
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
      dig[u] = sort_digit(a, keys[u]) - lo;
      const bool active = g0 + u * kWave + lane < w1 && (uint32_t)dig[u] < (uint32_t)a.width;
      pos[u] = bumped[u] = 0;
      if (active) {
        pos[u] = mine[dig[u]];
        bumped[u] = atomicAdd(&mine[dig[u]], 1);
      } else {
        dig[u] = -1;
      }
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const int d = dig[u];
      const bool active = d >= 0;
      uint64_t shared = __ballot(active && bumped[u] != pos[u]);   // the non-first lanes of shared bins
      while (shared) {
        const int l = __builtin_ctzll(shared);
        const int v = __shfl(d, l, kWave);
        const uint64_t grp = __ballot(d == v);                     // all lanes of that bin; they read the same base
        if (d == v) pos[u] += __popcll(grp & below);
        shared &= ~grp;
      }
      if (active) {
        if (a.keys_out) a.keys_out[pos[u]] = keys[u];
        a.vals_out[pos[u]] = vals[u];
        if (a.tok_out) a.tok_out[pos[u]] = (int32_t)(((uint64_t)(uint32_t)vals[u] * a.inv_top_k) >> a.inv_shift);   // val / top_k
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
  int passes, lo_bits, bins[2], width, stride, tile, tiles;
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
  pl->width = ((maxb + kSlices - 1) / kSlices + kBinChunk - 1) / kBinChunk * kBinChunk;
  pl->stride = pl->width * kSlices;
  // a wave places an eighth of a tile, 64 items a step: tiles of 8192 pairs are 16 steps; at most 256 tiles (a scatter
  // block sums its slice of every tile's row), more only where a tile would outgrow its 16-bit counters
  int64_t tile = 8192;
  if ((P + tile - 1) / tile > 256) tile = ((P + 255) / 256 + 1023) / 1024 * 1024;
  if (tile > kMaxTile) tile = kMaxTile;
  if ((P + tile - 1) / tile > kMaxSortTiles) return false;   // more than 64 Mi pairs
  pl->tile = (int)tile;
  pl->tiles = (int)((P + tile - 1) / tile);
  if (pl->tiles < 1) pl->tiles = 1;
  pl->hist_entries = (size_t)pl->stride * pl->tiles;
  return true;
}

}  // namespace omni

// workspace: hist [tiles][stride] u16 | slice sums [tiles][8] u32 | two-pass sorts only: keys A [P] | keys B [P] | pair ids [P]
extern "C" OMNI_API size_t omni_schedule_workspace_bytes(int64_t num_tokens, int32_t num_experts_per_token, int64_t num_experts) {
  using namespace omni;
  const int64_t P = num_tokens * (int64_t)num_experts_per_token;
  SortPlan pl;
  if (num_tokens < 0 || num_experts_per_token < 0 || num_experts <= 0 || !make_plan(P, num_experts, &pl)) return 0;
  return align_up(pl.hist_entries * 2, 256) + align_up((size_t)pl.tiles * kSlices * 4, 256) +
         (pl.passes == 2 ? 3 * align_up((size_t)P * 4 + 4, 256) : 0);
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
  uint32_t* slice_tot = (uint32_t*)w; w += align_up((size_t)pl.tiles * kSlices * 4, 256);
  int32_t* keys_a = (int32_t*)w;     w += align_up((size_t)P * 4 + 4, 256);      // the three arrays exist for two-pass sorts only
  int32_t* keys_b = (int32_t*)w;     w += align_up((size_t)P * 4 + 4, 256);
  int32_t* vals_a = (int32_t*)w;

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
      a.slice_tot = slice_tot;
      a.num_pairs = P;
      a.tile = pl.tile;
      a.tiles = pl.tiles;
      a.bins = pl.bins[pass];
      a.width = pl.width;
      a.stride = pl.stride;
      a.shift = pass == 0 ? 0 : pl.lo_bits;
      a.mask = (pl.passes == 2 && pass == 0) ? (uint32_t)((1 << pl.lo_bits) - 1) : 0xFFFFFFFFu;
      a.last = last ? 1 : 0;
      a.num_experts = (uint32_t)N;
      a.inv_shift = 30;
      while ((1ll << (a.inv_shift - 30)) < (int64_t)num_experts_per_token) ++a.inv_shift;
      a.inv_top_k = num_experts_per_token > 0 ? ((1ull << a.inv_shift) + num_experts_per_token - 1) / (uint64_t)num_experts_per_token : 0;
      hipLaunchKernelGGL(sort_count_kernel, dim3(a.tiles), dim3(kSortThreads), (size_t)a.stride * 4, s, a);
      hipLaunchKernelGGL(sort_scatter_kernel, dim3(a.tiles * kSlices), dim3(kSortThreads), 0, s, a);
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
