// Cartesian-product router selection for gfx950.
//
// Replaces the reference's two torch.topk launches plus its serial max/argmax
// Triton kernel (omni_moe/ops/triton/omni_router.py:8-95, 167-232).  One 64-lane
// wave owns one token and never leaves registers:
//   1. each half's r scores sit `R` per lane and are sorted descending by a bitonic
//      network (cross-lane exchanges for strides < 64, register exchanges above),
//      ordered by (score desc, key index asc) -- a total order, so ties resolve to
//      the lower key index;
//   2. candidate sums sx[a]+sy[b] are formed in the storage dtype, but only for the
//      cells with (a+1)(b+1) <= k: both half lists are sorted, so a cell (a,b) is
//      preceded by the (a+1)(b+1)-1 cells it is dominated by (each has a score >= its
//      own and a lower position a*k'+b), and cannot be among the first k otherwise.
//      That is 50 cells instead of 256 at k=16, 119 instead of 1024 at k=32;
//   3. the candidates are sorted by (score desc, position asc) with the same
//      network and the first k are written out with id = ix[a]*r + iy[b].
#include "common.h"
#include "omni_moe_hip.h"

// defined beside the GEMM kernels: z = x [Wx;Wy]^T, optionally with per-32-row column
// partial statistics (mean, M2) [ceil(T/32)][2r] of the rounded z
int omni_gemm_router_projection(const void* x, const void* wx, const void* wy, void* z, float* part_mean, float* part_m2,
                                int64_t T, int H, int r, int dtype, void* stream);

namespace omni {

// strict "a goes before b": higher score first, then lower payload
__device__ __forceinline__ bool goes_before(float sa, int pa, float sb, int pb) {
  return (sa > sb) || (sa == sb && pa < pb);
}

// Compare-exchange step with a compile-time lane distance, fully unrolled (small R only).
template <int R, int SIZE, int STRIDE>
__device__ __forceinline__ void lane_stage_ct(float (&s)[R], int (&p)[R], const int lane) {
#pragma unroll
  for (int a = 0; a < R; ++a) {
    const float os = xor_lane_f<STRIDE>(s[a], lane);
    const int op = xor_lane_i<STRIDE>(p[a], lane);
    const bool up = (((a * kWave) | lane) & SIZE) == 0;
    const bool lower = (lane & STRIDE) == 0;
    const bool take_other = (lower == up) != goes_before(s[a], p[a], os, op);
    s[a] = take_other ? os : s[a];
    p[a] = take_other ? op : p[a];
  }
}
// strides STRIDE, STRIDE/2, ..., 1 of the merge for block size SIZE, on NL lists in lockstep
template <int R, int SIZE, int STRIDE>
__device__ __forceinline__ void lane_stages_ct(float (&s0)[R], int (&p0)[R], float (&s1)[R], int (&p1)[R], const int lane, const bool two) {
  if constexpr (STRIDE >= 1) {
    lane_stage_ct<R, SIZE, STRIDE>(s0, p0, lane);
    if (two) lane_stage_ct<R, SIZE, STRIDE>(s1, p1, lane);
    lane_stages_ct<R, SIZE, STRIDE / 2>(s0, p0, s1, p1, lane, two);
  }
}
template <int R, int SIZE>
__device__ __forceinline__ void small_sizes_ct(float (&s0)[R], int (&p0)[R], float (&s1)[R], int (&p1)[R], const int lane, const bool two) {
  if constexpr (SIZE <= kWave) {
    lane_stages_ct<R, SIZE, SIZE / 2>(s0, p0, s1, p1, lane, two);
    small_sizes_ct<R, SIZE * 2>(s0, p0, s1, p1, lane, two);
  }
}

// One compare-exchange step between lanes `stride` apart (stride < 64), all R registers.
template <int R>
__device__ __forceinline__ void lane_stage(float (&s)[R], int (&p)[R], const int lane, const int size, const int stride) {
#pragma unroll
  for (int a = 0; a < R; ++a) {
    const float os = __shfl_xor(s[a], stride, kWave);
    const int op = __shfl_xor(p[a], stride, kWave);
    const bool up = (((a * kWave) | lane) & size) == 0;
    const bool lower = (lane & stride) == 0;
    const bool take_other = (lower == up) != goes_before(s[a], p[a], os, op);
    s[a] = take_other ? os : s[a];
    p[a] = take_other ? op : p[a];
  }
}

// One compare-exchange step between registers RS apart (element stride 64*RS).
template <int R, int SIZE, int RS>
__device__ __forceinline__ void reg_stage(float (&s)[R], int (&p)[R]) {
#pragma unroll
  for (int a = 0; a < R; ++a) {
    if ((a & RS) == 0) {
      const int b = a | RS;
      const bool up = ((a * kWave) & SIZE) == 0;
      const bool swap = goes_before(s[a], p[a], s[b], p[b]) != up;
      const float ts = swap ? s[b] : s[a];
      const int tp = swap ? p[b] : p[a];
      s[b] = swap ? s[a] : s[b];
      p[b] = swap ? p[a] : p[b];
      s[a] = ts;
      p[a] = tp;
    }
  }
}

template <int R, int SIZE, int RS>
__device__ __forceinline__ void reg_stages_down(float (&s)[R], int (&p)[R]) {
  if constexpr (RS >= 1) {
    reg_stage<R, SIZE, RS>(s, p);
    reg_stages_down<R, SIZE, RS / 2>(s, p);
  }
}

// Merge steps for block size SIZE (> 64) and the sizes above it, up to 64*R.
constexpr int kUnrollMaxR = 2;     // lists of <= 128 items use the unrolled, LDS-free exchanges

template <int R, int SIZE>
__device__ __forceinline__ void big_sizes(float (&s)[R], int (&p)[R], const int lane) {
  if constexpr (SIZE <= kWave * R) {
    reg_stages_down<R, SIZE, SIZE / (2 * kWave)>(s, p);
    if constexpr (R <= kUnrollMaxR) {
      lane_stages_ct<R, SIZE, kWave / 2>(s, p, s, p, lane, false);
    } else {
#pragma nounroll
      for (int stride = kWave / 2; stride >= 1; stride >>= 1) lane_stage<R>(s, p, lane, SIZE, stride);
    }
    big_sizes<R, SIZE * 2>(s, p, lane);
  }
}

// Sorts the 64*R (score, payload) items held as item e = reg*64 + lane with a bitonic
// network.  Steps between lanes run as rolled loops (the shuffle distance is a run-time
// value); steps between registers are unrolled so that register indices are constants.
template <int R>
__device__ __forceinline__ void bitonic_sort(float (&s)[R], int (&p)[R], const int lane) {
  if constexpr (R <= kUnrollMaxR) {
    small_sizes_ct<R, 2>(s, p, s, p, lane, false);
  } else {
#pragma nounroll
    for (int size = 2; size <= kWave; size <<= 1) {
#pragma nounroll
      for (int stride = size >> 1; stride >= 1; stride >>= 1) lane_stage<R>(s, p, lane, size, stride);
    }
  }
  big_sizes<R, 2 * kWave>(s, p, lane);
}

// Two independent lists sorted in lockstep: the two dependency chains interleave, which
// hides most of the cross-lane exchange latency.
template <int R, int SIZE>
__device__ __forceinline__ void big_sizes2(float (&s0)[R], int (&p0)[R], float (&s1)[R], int (&p1)[R], const int lane) {
  if constexpr (SIZE <= kWave * R) {
    reg_stages_down<R, SIZE, SIZE / (2 * kWave)>(s0, p0);
    reg_stages_down<R, SIZE, SIZE / (2 * kWave)>(s1, p1);
    if constexpr (R <= kUnrollMaxR) {
      lane_stages_ct<R, SIZE, kWave / 2>(s0, p0, s1, p1, lane, true);
    } else {
#pragma nounroll
      for (int stride = kWave / 2; stride >= 1; stride >>= 1) {
        lane_stage<R>(s0, p0, lane, SIZE, stride);
        lane_stage<R>(s1, p1, lane, SIZE, stride);
      }
    }
    big_sizes2<R, SIZE * 2>(s0, p0, s1, p1, lane);
  }
}
template <int R>
__device__ __forceinline__ void bitonic_sort2(float (&s0)[R], int (&p0)[R], float (&s1)[R], int (&p1)[R], const int lane) {
  if constexpr (R <= kUnrollMaxR) {
    small_sizes_ct<R, 2>(s0, p0, s1, p1, lane, true);
  } else {
#pragma nounroll
    for (int size = 2; size <= kWave; size <<= 1) {
#pragma nounroll
      for (int stride = size >> 1; stride >= 1; stride >>= 1) {
        lane_stage<R>(s0, p0, lane, size, stride);
        lane_stage<R>(s1, p1, lane, size, stride);
      }
    }
  }
  big_sizes2<R, 2 * kWave>(s0, p0, s1, p1, lane);
}

// value of sorted item `i` (i < 128) of a list held as item = reg*64+lane
template <int R, typename T>
__device__ __forceinline__ T sorted_item(const T (&v)[R], int i) {
  T r0 = __shfl(v[0], i & 63, kWave);
  if constexpr (R >= 2) {
    T r1 = __shfl(v[1], i & 63, kWave);
    r0 = (i >= kWave) ? r1 : r0;
  }
  return r0;
}

// Storage dtype handled at run time (one uniform branch per access) to keep the number of
// kernel instantiations at |R| x |C|.
__device__ __forceinline__ float load_score(const void* p, int64_t i, int dt) {
  return dt == kBF16 ? Elem<kBF16>::load(p, i) : dt == kF16 ? Elem<kF16>::load(p, i) : Elem<kF32>::load(p, i);
}
__device__ __forceinline__ float round_score(float v, int dt) {
  return dt == kBF16 ? Elem<kBF16>::round(v) : dt == kF16 ? Elem<kF16>::round(v) : v;
}
__device__ __forceinline__ void store_score(void* p, int64_t i, float v, int dt) {
  if (dt == kBF16) Elem<kBF16>::store(p, i, v);
  else if (dt == kF16) Elem<kF16>::store(p, i, v);
  else Elem<kF32>::store(p, i, v);
}

constexpr int kRouterWaves = 4;
constexpr int kMaxKeys = 1024;        // keys per half that the select kernels hold in registers (16 per lane)
constexpr int kMaxKeysChunked = 16384; // ... that the chunked kernel walks (16-bit scores, at most 64 candidates per half)
constexpr float kNegInf = -__builtin_huge_valf();

struct SelectArgs {
  const void* lx;        // x-half scores of token t at lx[t*row_stride + key]
  const void* ly;
  int64_t row_stride;
  const float* stats;    // NULL, or [4][r] fp32: mean_x, rstd_x, mean_y, rstd_y -> the inputs are raw
                         // projections; normalise and log-softmax them before selecting
  const void* run_mean[2];  // instead of stats (eval-mode BatchNorm): the two halves' running_mean / running_var
  const void* run_var[2];   //   [r] of dtype stat_dt; mean and 1/sqrt(var + eps) are formed here, and block 0
  float* stats_out;         //   also leaves them at stats_out [4][r] (may be NULL) for a backward pass
  int stat_dt;
  float eps;
  void* scores;          // [T,k] storage dtype, may be NULL
  void* gates;           // [T,k] storage dtype = exp(score), may be NULL
  int32_t* indices;      // [T,k]
  int num_tokens, r, k, kp, dt;
  uint8_t row_cells[128]; // candidate cells in row a: min(kp, k/(a+1)), filled by select_dispatch
  int64_t* count_batch[2]; // NULL, or BatchNorm's num_batches_tracked of the two halves: incremented here, behind the
                           // kernel that read them (train-mode router stage)
};

__device__ __forceinline__ void count_batch(const SelectArgs& g) {
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (g.count_batch[0]) *g.count_batch[0] += 1;
    if (g.count_batch[1]) *g.count_batch[1] += 1;
  }
  if (blockIdx.x == 0 && !g.stats && g.run_mean[0] && g.stats_out) {   // eval mode: the statistics a backward pass reads
    for (int i = threadIdx.x; i < 2 * g.r; i += blockDim.x) {
      const int half = i >= g.r, key = i - half * g.r;
      g.stats_out[(2 * half) * g.r + key] = load_score(g.run_mean[half], key, g.stat_dt);
      g.stats_out[(2 * half + 1) * g.r + key] = __builtin_amdgcn_rsqf(load_score(g.run_var[half], key, g.stat_dt) + g.eps);
    }
  }
}

// BatchNorm (affine-free) of one raw projection value, rounded to the storage dtype as the reference's BatchNorm output is
__device__ __forceinline__ float normalise_one(float v, const SelectArgs& g, const int half, const int key, const int r, const int dt) {
  float mean, rstd;
  if (g.stats) {
    mean = g.stats[(2 * half) * r + key];
    rstd = g.stats[(2 * half + 1) * r + key];
  } else {
    mean = load_score(g.run_mean[half], key, g.stat_dt);
    rstd = __builtin_amdgcn_rsqf(load_score(g.run_var[half], key, g.stat_dt) + g.eps);
  }
  return round_score((v - mean) * rstd, dt);
}

// BatchNorm (affine-free) then log-softmax of one half, in place: v holds the raw projection
// of key a*64+lane (NaN-free -inf padding past r).  Each stage rounds to the storage dtype
// where the reference's torch ops do (BN output, log-softmax output; omni_moe.py:70-78).
template <int R>
__device__ __forceinline__ void normalise_half(float (&v)[R], const SelectArgs& g, const int half, int r, int lane, int dt) {
  float m = kNegInf;
#pragma unroll
  for (int a = 0; a < R; ++a) {
    const int key = a * kWave + lane;
    if (key < r) {
      float mean, rstd;
      if (g.stats) {
        mean = g.stats[(2 * half) * r + key];
        rstd = g.stats[(2 * half + 1) * r + key];
      } else {                                   // per token and key: the hardware's reciprocal square root (1 ulp), as in stats_out
        mean = load_score(g.run_mean[half], key, g.stat_dt);
        rstd = __builtin_amdgcn_rsqf(load_score(g.run_var[half], key, g.stat_dt) + g.eps);
      }
      v[a] = round_score((v[a] - mean) * rstd, dt);
    }
    m = fmaxf(m, v[a]);
  }
  m = wave_max(m);
  float e = 0.f;
#pragma unroll
  for (int a = 0; a < R; ++a) e += (a * kWave + lane < r) ? expf(v[a] - m) : 0.f;
  const float lse = logf(wave_sum(e));
#pragma unroll
  for (int a = 0; a < R; ++a)
    if (a * kWave + lane < r) v[a] = round_score(v[a] - m - lse, dt);
}

// This lane's candidate cells: cell index ci = c*64+lane enumerates rows a = 0..kp-1 with
// min(kp, k/(a+1)) cells each.  Payload (a<<8)|b orders like position a*kp+b.  The row counts
// come with the arguments: the lanes fetch them all at once (row a in lane a%64) and the uniform
// loop hands them round by readlane, so it waits for memory once, not once per row.
template <int R, int C>
__device__ __forceinline__ void candidate_cells(int (&cell)[C], const SelectArgs& g, const int kp, const int lane) {
#pragma unroll
  for (int c = 0; c < C; ++c) cell[c] = -1;
  // Measured per shape: with 4 or 8 keys and fewer than 8 cells per lane the plain loop, one load per row, is the faster
  // one by 3-6 % of the kernel (32768 tokens, 256-512 keys per half, k = 32); everywhere else the lanes' loop is, by 1-6 %.
  if constexpr (R > 2 && C < 8) {
    for (int a = 0, start = 0; a < kp; ++a) {
      const int cnt = g.row_cells[a];
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const int b = c * kWave + lane - start;
        cell[c] = (unsigned)b < (unsigned)cnt ? (a << 8) | b : cell[c];
      }
      start += cnt;
    }
    return;
  }
  const int cnt_lo = lane < kp ? g.row_cells[lane] : 0;
  const int cnt_hi = lane + kWave < kp ? g.row_cells[lane + kWave] : 0;
  int start = 0;
  for (int a = 0; a < min(kp, kWave); ++a) {
    const int cnt = __builtin_amdgcn_readlane(cnt_lo, a);
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const int b = c * kWave + lane - start;
      cell[c] = (unsigned)b < (unsigned)cnt ? (a << 8) | b : cell[c];
    }
    start += cnt;
  }
  for (int a = kWave; a < kp; ++a) {
    const int cnt = __builtin_amdgcn_readlane(cnt_hi, a - kWave);
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const int b = c * kWave + lane - start;
      cell[c] = (unsigned)b < (unsigned)cnt ? (a << 8) | b : cell[c];
    }
    start += cnt;
  }
}

// R = half keys per lane (r <= 64*R); C = candidate cells per lane.  With few keys per lane a wave requests
// the raw scores of its first token before anything else and those of its next token as soon as the current
// token's are consumed.
template <int R, int C>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_select_kernel(const SelectArgs g) {
  count_batch(g);
  const int lane = lane_id();
  const int wave = blockIdx.x * kRouterWaves + (threadIdx.x >> 6);
  const int num_waves = gridDim.x * kRouterWaves;
  const int r = g.r, k = g.k, kp = g.kp, dt = g.dt;

  float rx[R], ry[R];                             // raw scores of the token about to be selected
  auto load_raw = [&](int t) __attribute__((always_inline)) {
#pragma unroll
    for (int a = 0; a < R; ++a) {
      const int key = a * kWave + lane;
      const bool ok = key < r;
      rx[a] = ok ? load_score(g.lx, int64_t(t) * g.row_stride + key, dt) : kNegInf;
      ry[a] = ok ? load_score(g.ly, int64_t(t) * g.row_stride + key, dt) : kNegInf;
    }
  };
  constexpr bool kPrefetch = R <= 2;              // beyond that the extra live registers cost a wave per SIMD
  if (kPrefetch && wave < g.num_tokens) load_raw(wave);
  int cell[C];
  candidate_cells<R, C>(cell, g, kp, lane);

  for (int t = wave; t < g.num_tokens; t += num_waves) {
    float sx[R], sy[R];
    int px[R], py[R];
#pragma unroll
    for (int a = 0; a < R; ++a) {
      const int key = a * kWave + lane;
      const bool ok = key < r;
      sx[a] = kPrefetch ? rx[a] : ok ? load_score(g.lx, int64_t(t) * g.row_stride + key, dt) : kNegInf;
      sy[a] = kPrefetch ? ry[a] : ok ? load_score(g.ly, int64_t(t) * g.row_stride + key, dt) : kNegInf;
      px[a] = py[a] = key;
    }
    if (kPrefetch && t + num_waves < g.num_tokens) load_raw(t + num_waves);
    if (g.stats || g.run_mean[0]) {
      normalise_half<R>(sx, g, 0, r, lane, dt);
      normalise_half<R>(sy, g, 1, r, lane, dt);
    }
    bitonic_sort2<R>(sx, px, sy, py, lane);

    float cs[C];
    int cp[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const bool ok = cell[c] >= 0;
      const int a = ok ? (cell[c] >> 8) : 0, b = ok ? (cell[c] & 255) : 0;
      const float va = sorted_item<R>(sx, a), vb = sorted_item<R>(sy, b);
      cs[c] = ok ? round_score(va + vb, dt) : kNegInf;
      cp[c] = ok ? cell[c] : (0x40000000 | (c * kWave + lane));
    }
    bitonic_sort<C>(cs, cp, lane);

    constexpr int kOut = (C >= 2) ? 2 : 1;          // k <= 128 -> winners live in regs 0..1
#pragma unroll
    for (int c = 0; c < kOut; ++c) {
      const int j = c * kWave + lane;
      const bool ok = j < k;
      const int a = ok ? (cp[c] >> 8) & 255 : 0, b = ok ? (cp[c] & 255) : 0;
      const int ia = sorted_item<R>(px, a), ib = sorted_item<R>(py, b);
      if (ok) {
        const int64_t o = int64_t(t) * k + j;
        if (g.scores) store_score(g.scores, o, cs[c], dt);
        if (g.gates) store_score(g.gates, o, expf(cs[c]), dt);      // gate = P(x key) * P(y key)
        g.indices[o] = ia * r + ib;
      }
    }
  }
}

// ---- 16-bit scores: (score, payload) packed into one ordered 32-bit key ---------------------
// key = order-preserving image of the 16-bit score << 16 | (0xFFFF - payload): a larger key goes
// first, equal scores resolve to the lower payload, and a compare-exchange is one max / min.
// Four times fewer VALU instructions than the (float, int) pairs the fp32 path needs.
__device__ __forceinline__ uint32_t ord16(uint32_t bits) { return bits ^ ((bits & 0x8000u) ? 0xFFFFu : 0x8000u); }
__device__ __forceinline__ uint32_t unord16(uint32_t u) { return u ^ ((u & 0x8000u) ? 0x8000u : 0xFFFFu); }
__device__ __forceinline__ uint32_t make_key(float v, int payload, int dt) {      // v is representable in dt
  v += 0.0f;                                                                      // -0 -> +0: they compare equal as floats
  const uint32_t bits = dt == kBF16 ? (uint32_t)f32_to_bf16_bits(v) : (uint32_t)f32_to_f16_bits(v);
  return (ord16(bits) << 16) | (0xFFFFu - (uint32_t)payload);
}
__device__ __forceinline__ float key_score(uint32_t key, int dt) {
  const uint32_t bits = unord16(key >> 16);
  return dt == kBF16 ? bf16_bits_to_f32((uint16_t)bits) : f16_bits_to_f32((uint16_t)bits);
}
__device__ __forceinline__ int key_payload(uint32_t key) { return (int)(0xFFFFu - (key & 0xFFFFu)); }

template <int R, int SIZE, int STRIDE>
__device__ __forceinline__ void kstage_ct(uint32_t (&k)[R], const int lane) {
#pragma unroll
  for (int a = 0; a < R; ++a) {
    const uint32_t o = (uint32_t)xor_lane_i<STRIDE>((int)k[a], lane);
    const bool up = (((a * kWave) | lane) & SIZE) == 0, lower = (lane & STRIDE) == 0;
    k[a] = (lower == up) ? max(k[a], o) : min(k[a], o);
  }
}
template <int R>
__device__ __forceinline__ void kstage_rt(uint32_t (&k)[R], const int lane, const int size, const int stride) {
#pragma unroll
  for (int a = 0; a < R; ++a) {
    const uint32_t o = (uint32_t)__shfl_xor((int)k[a], stride, kWave);
    const bool up = (((a * kWave) | lane) & size) == 0, lower = (lane & stride) == 0;
    k[a] = (lower == up) ? max(k[a], o) : min(k[a], o);
  }
}
template <int R, int SIZE, int RS>
__device__ __forceinline__ void kreg_stages(uint32_t (&k)[R]) {
  if constexpr (RS >= 1) {
#pragma unroll
    for (int a = 0; a < R; ++a) {
      if ((a & RS) == 0) {
        const int b = a | RS;
        const bool up = ((a * kWave) & SIZE) == 0;
        const uint32_t hi = max(k[a], k[b]), lo = min(k[a], k[b]);
        k[a] = up ? hi : lo;
        k[b] = up ? lo : hi;
      }
    }
    kreg_stages<R, SIZE, RS / 2>(k);
  }
}
// lane distances STRIDE..1 of the merge for block size SIZE, on one or two lists
template <int R, int SIZE, int STRIDE>
__device__ __forceinline__ void kstages_ct(uint32_t (&k0)[R], uint32_t (&k1)[R], const int lane, const bool two) {
  if constexpr (STRIDE >= 1) {
    kstage_ct<R, SIZE, STRIDE>(k0, lane);
    if (two) kstage_ct<R, SIZE, STRIDE>(k1, lane);
    kstages_ct<R, SIZE, STRIDE / 2>(k0, k1, lane, two);
  }
}
template <int R, int SIZE>
__device__ __forceinline__ void ksizes(uint32_t (&k0)[R], uint32_t (&k1)[R], const int lane, const bool two) {
  if constexpr (SIZE <= kWave * R) {
    if constexpr (SIZE > kWave) {
      kreg_stages<R, SIZE, SIZE / (2 * kWave)>(k0);
      if (two) kreg_stages<R, SIZE, SIZE / (2 * kWave)>(k1);
    }
    constexpr int kFirst = SIZE > kWave ? kWave / 2 : SIZE / 2;
    if constexpr (R <= kUnrollMaxR) {
      kstages_ct<R, SIZE, kFirst>(k0, k1, lane, two);
    } else {
#pragma nounroll
      for (int stride = kFirst; stride >= 1; stride >>= 1) {
        kstage_rt<R>(k0, lane, SIZE, stride);
        if (two) kstage_rt<R>(k1, lane, SIZE, stride);
      }
    }
    ksizes<R, SIZE * 2>(k0, k1, lane, two);
  }
}
// sorts the 64*R keys of each list descending (item e = reg*64 + lane)
template <int R> __device__ __forceinline__ void ksort(uint32_t (&k)[R], const int lane) { ksizes<R, 2>(k, k, lane, false); }
template <int R> __device__ __forceinline__ void ksort2(uint32_t (&k0)[R], uint32_t (&k1)[R], const int lane) { ksizes<R, 2>(k0, k1, lane, true); }

// The 64 largest keys of each list (64*R keys, item = reg*64 + lane), descending, into register 0 -- all that the
// candidate stage reads when k' <= 64.  Every register is sorted across the lanes by itself (compile-time lane
// distances, no LDS), then the registers are merged pairwise: for two descending runs A and B, max(A[i], B[63-i])
// holds the 64 largest of both as a bitonic sequence, which six more compare-exchange steps put in order.  About a
// third of the compare-exchanges of a full sort of 512 keys, and none of them through run-time lane distances.
template <int R>
__device__ __forceinline__ void ktop64_2(uint32_t (&k0)[R], uint32_t (&k1)[R], const int lane) {
#pragma unroll
  for (int a = 0; a < R; ++a) {
    uint32_t x[1] = {k0[a]}, y[1] = {k1[a]};
    ksizes<1, 2>(x, y, lane, true);
    k0[a] = x[0];
    k1[a] = y[0];
  }
#pragma unroll
  for (int width = R; width > 1; width /= 2) {
#pragma unroll
    for (int a = 0; a < width / 2; ++a) {
      uint32_t x[1] = {max(k0[a], (uint32_t)__shfl((int)k0[a + width / 2], 63 - lane, kWave))};
      uint32_t y[1] = {max(k1[a], (uint32_t)__shfl((int)k1[a + width / 2], 63 - lane, kWave))};
      kstages_ct<1, kWave, kWave / 2>(x, y, lane, true);
      k0[a] = x[0];
      k1[a] = y[0];
    }
  }
}

template <int R>
__device__ __forceinline__ uint32_t sorted_key(const uint32_t (&v)[R], int i) {
  uint32_t r0 = (uint32_t)__shfl((int)v[0], i & 63, kWave);
  if constexpr (R >= 2) {
    const uint32_t r1 = (uint32_t)__shfl((int)v[1], i & 63, kWave);
    r0 = (i >= kWave) ? r1 : r0;
  }
  return r0;
}

// Same selection as router_select_kernel for bf16 / f16 storage, on packed keys.
template <int R, int C>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_select_packed_kernel(const SelectArgs g) {
  count_batch(g);
  const int lane = lane_id();
  const int wave = blockIdx.x * kRouterWaves + (threadIdx.x >> 6);
  const int num_waves = gridDim.x * kRouterWaves;
  const int r = g.r, k = g.k, kp = g.kp, dt = g.dt;

  float rx[R], ry[R];                             // as in router_select_kernel
  auto load_raw = [&](int t) __attribute__((always_inline)) {
#pragma unroll
    for (int a = 0; a < R; ++a) {
      const int key = a * kWave + lane;
      const bool ok = key < r;
      rx[a] = ok ? load_score(g.lx, int64_t(t) * g.row_stride + key, dt) : kNegInf;
      ry[a] = ok ? load_score(g.ly, int64_t(t) * g.row_stride + key, dt) : kNegInf;
    }
  };
  constexpr bool kPrefetch = R <= 2;              // beyond that the extra live registers cost a wave per SIMD
  if (kPrefetch && wave < g.num_tokens) load_raw(wave);
  int cell[C];
  candidate_cells<R, C>(cell, g, kp, lane);

  for (int t = wave; t < g.num_tokens; t += num_waves) {
    float sx[R], sy[R];
#pragma unroll
    for (int a = 0; a < R; ++a) {
      const int key = a * kWave + lane;
      const bool ok = key < r;
      sx[a] = kPrefetch ? rx[a] : ok ? load_score(g.lx, int64_t(t) * g.row_stride + key, dt) : kNegInf;
      sy[a] = kPrefetch ? ry[a] : ok ? load_score(g.ly, int64_t(t) * g.row_stride + key, dt) : kNegInf;
    }
    if (kPrefetch && t + num_waves < g.num_tokens) load_raw(t + num_waves);
    if (g.stats || g.run_mean[0]) {
      normalise_half<R>(sx, g, 0, r, lane, dt);
      normalise_half<R>(sy, g, 1, r, lane, dt);
    }
    uint32_t kx[R], ky[R];
#pragma unroll
    for (int a = 0; a < R; ++a) {
      const int key = a * kWave + lane;
      kx[a] = key < r ? make_key(sx[a], key, dt) : 0u;          // 0 sorts behind every real key
      ky[a] = key < r ? make_key(sy[a], key, dt) : 0u;
    }
    if (R > kUnrollMaxR && kp <= kWave) ktop64_2<R>(kx, ky, lane);    // uniform: kp comes with the arguments
    else ksort2<R>(kx, ky, lane);

    uint32_t ck[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const bool ok = cell[c] >= 0;
      const int a = ok ? (cell[c] >> 8) : 0, b = ok ? (cell[c] & 255) : 0;
      const float va = key_score(sorted_key<R>(kx, a), dt), vb = key_score(sorted_key<R>(ky, b), dt);
      ck[c] = ok ? make_key(round_score(va + vb, dt), cell[c], dt) : 0u;
    }
    ksort<C>(ck, lane);

    constexpr int kOut = (C >= 2) ? 2 : 1;          // k <= 128 -> winners live in regs 0..1
#pragma unroll
    for (int c = 0; c < kOut; ++c) {
      const int j = c * kWave + lane;
      const bool ok = j < k;
      const int pl = ok ? key_payload(ck[c]) : 0;
      const int ia = key_payload(sorted_key<R>(kx, pl >> 8)), ib = key_payload(sorted_key<R>(ky, pl & 255));
      if (ok) {
        const int64_t o = int64_t(t) * k + j;
        const float sc = key_score(ck[c], dt);
        if (g.scores) store_score(g.scores, o, sc, dt);
        if (g.gates) store_score(g.gates, o, expf(sc), dt);         // gate = P(x key) * P(y key)
        g.indices[o] = ia * r + ib;
      }
    }
  }
}

// More keys per half than a wave's registers hold (r > 1024): 16-bit scores, k' <= 64.  The row is walked in chunks of
// 512 keys per half: each chunk's 64 best (ktop64_2) are merged into the running 64 best by the same max(A[i], B[63-i])
// step.  With the BatchNorm + log-softmax front the row is read three times (maximum, sum of exponentials, keys), each
// time with the arithmetic and the per-lane summation order of normalise_half, so a row gives the bits it would give there.
template <int C>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_select_chunked_kernel(const SelectArgs g) {
  constexpr int RC = 8, kChunk = RC * kWave;
  count_batch(g);
  const int lane = lane_id();
  const int wave = blockIdx.x * kRouterWaves + (threadIdx.x >> 6);
  const int num_waves = gridDim.x * kRouterWaves;
  const int r = g.r, k = g.k, kp = g.kp, dt = g.dt;
  const int chunks = (r + kChunk - 1) / kChunk;
  const bool norm = g.stats || g.run_mean[0];
  int cell[C];
  candidate_cells<1, C>(cell, g, kp, lane);

  for (int t = wave; t < g.num_tokens; t += num_waves) {
    const int64_t row = int64_t(t) * g.row_stride;
    float mx[2] = {0.f, 0.f}, lse[2] = {0.f, 0.f};
    if (norm) {
      for (int half = 0; half < 2; ++half) {
        const void* src = half ? g.ly : g.lx;
        float m = kNegInf;
        for (int c = 0; c < chunks; ++c)
#pragma unroll
          for (int a = 0; a < RC; ++a) {
            const int key = c * kChunk + a * kWave + lane;
            if (key < r) m = fmaxf(m, normalise_one(load_score(src, row + key, dt), g, half, key, r, dt));
          }
        m = wave_max(m);
        float e = 0.f;
        for (int c = 0; c < chunks; ++c)
#pragma unroll
          for (int a = 0; a < RC; ++a) {
            const int key = c * kChunk + a * kWave + lane;
            e += key < r ? expf(normalise_one(load_score(src, row + key, dt), g, half, key, r, dt) - m) : 0.f;
          }
        mx[half] = m;
        lse[half] = logf(wave_sum(e));
      }
    }
    uint32_t bx = 0u, by = 0u;                      // the 64 best keys so far of each half, descending across the lanes
    for (int c = 0; c < chunks; ++c) {
      uint32_t kx[RC], ky[RC];
#pragma unroll
      for (int a = 0; a < RC; ++a) {
        const int key = c * kChunk + a * kWave + lane;
        const bool ok = key < r;
        float vx = ok ? load_score(g.lx, row + key, dt) : 0.f, vy = ok ? load_score(g.ly, row + key, dt) : 0.f;
        if (norm && ok) {
          vx = round_score(normalise_one(vx, g, 0, key, r, dt) - mx[0] - lse[0], dt);
          vy = round_score(normalise_one(vy, g, 1, key, r, dt) - mx[1] - lse[1], dt);
        }
        kx[a] = ok ? make_key(vx, key, dt) : 0u;    // 0 sorts behind every real key
        ky[a] = ok ? make_key(vy, key, dt) : 0u;
      }
      ktop64_2<RC>(kx, ky, lane);
      uint32_t x[1] = {max(bx, (uint32_t)__shfl((int)kx[0], 63 - lane, kWave))};
      uint32_t y[1] = {max(by, (uint32_t)__shfl((int)ky[0], 63 - lane, kWave))};
      kstages_ct<1, kWave, kWave / 2>(x, y, lane, true);
      bx = c == 0 ? kx[0] : x[0];
      by = c == 0 ? ky[0] : y[0];
    }
    const uint32_t sx[1] = {bx}, sy[1] = {by};

    uint32_t ck[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const bool ok = cell[c] >= 0;
      const int a = ok ? (cell[c] >> 8) : 0, b = ok ? (cell[c] & 255) : 0;
      const float va = key_score(sorted_key<1>(sx, a), dt), vb = key_score(sorted_key<1>(sy, b), dt);
      ck[c] = ok ? make_key(round_score(va + vb, dt), cell[c], dt) : 0u;
    }
    ksort<C>(ck, lane);

    constexpr int kOut = (C >= 2) ? 2 : 1;
#pragma unroll
    for (int c = 0; c < kOut; ++c) {
      const int j = c * kWave + lane;
      const bool ok = j < k;
      const int pl = ok ? key_payload(ck[c]) : 0;
      const int ia = key_payload(sorted_key<1>(sx, pl >> 8)), ib = key_payload(sorted_key<1>(sy, pl & 255));
      if (ok) {
        const int64_t o = int64_t(t) * k + j;
        const float sc = key_score(ck[c], dt);
        if (g.scores) store_score(g.scores, o, sc, dt);
        if (g.gates) store_score(g.gates, o, expf(sc), dt);
        g.indices[o] = ia * r + ib;
      }
    }
  }
}

template <int C>
static hipError_t launch_select_chunked(const SelectArgs& g, hipStream_t s) {
  int64_t blocks = ((int64_t)g.num_tokens + kRouterWaves - 1) / kRouterWaves;
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipLaunchKernelGGL((router_select_chunked_kernel<C>), dim3((unsigned)blocks), dim3(kRouterWaves * kWave), 0, s, g);
  return hipGetLastError();
}

// What the select kernels take: r <= 1024 with every dtype and k <= 128; beyond that 16-bit scores with k <= 64.
bool select_covers(int r, int k, int dtype) {
  if (r <= kMaxKeys) return true;
  return r <= kMaxKeysChunked && dtype != kF32 && k <= kWave;
}

static int num_cells(int k, int kp) {
  int n = 0;
  for (int a = 0; a < kp; ++a) n += (kp < k / (a + 1)) ? kp : k / (a + 1);
  return n;
}

template <int R, int C>
static hipError_t launch_select(const SelectArgs& g, hipStream_t s) {
  int64_t blocks = ((int64_t)g.num_tokens + kRouterWaves - 1) / kRouterWaves;
  if (blocks > 256 * 16) blocks = 256 * 16;     // waves loop over tokens beyond that
  if (g.dt == kF32)
    hipLaunchKernelGGL((router_select_kernel<R, C>), dim3((unsigned)blocks), dim3(kRouterWaves * kWave), 0, s, g);
  else
    hipLaunchKernelGGL((router_select_packed_kernel<R, C>), dim3((unsigned)blocks), dim3(kRouterWaves * kWave), 0, s, g);
  return hipGetLastError();
}

template <int R>
static hipError_t select_by_cells(int cpl, const SelectArgs& g, hipStream_t s) {
  if (cpl <= 1) return launch_select<R, 1>(g, s);
  if (cpl <= 2) return launch_select<R, 2>(g, s);
  if (cpl <= 4) return launch_select<R, 4>(g, s);
  if (cpl <= 8) return launch_select<R, 8>(g, s);
  return launch_select<R, 16>(g, s);
}

static int select_dispatch(SelectArgs g, hipStream_t s) {
  g.kp = g.r < g.k ? g.r : g.k;
  for (int a = 0; a < 128; ++a) g.row_cells[a] = a < g.kp ? (uint8_t)(g.kp < g.k / (a + 1) ? g.kp : g.k / (a + 1)) : 0;
  const int cpl = (num_cells(g.k, g.kp) + kWave - 1) / kWave;   // <= 11 for k <= 128
  const int rpl = (g.r + kWave - 1) / kWave;
  hipError_t err;
  if (rpl <= 1) err = select_by_cells<1>(cpl, g, s);
  else if (rpl <= 2) err = select_by_cells<2>(cpl, g, s);
  else if (rpl <= 4) err = select_by_cells<4>(cpl, g, s);
  else if (rpl <= 8) err = select_by_cells<8>(cpl, g, s);
  else if (rpl <= 16) err = select_by_cells<16>(cpl, g, s);
  else if (!select_covers(g.r, g.k, g.dt)) return OMNI_ERR_UNSUPPORTED;   // the entry points refuse it before anything is enqueued
  else if (cpl <= 1) err = launch_select_chunked<1>(g, s);
  else if (cpl <= 2) err = launch_select_chunked<2>(g, s);
  else if (cpl <= 4) err = launch_select_chunked<4>(g, s);
  else err = launch_select_chunked<8>(g, s);                // k <= 64: at most 280 cells
  return err == hipSuccess ? OMNI_OK : OMNI_ERR_HIP_BASE + (int)err;
}

// ---- BatchNorm1d(affine=False) statistics over the T rows of z [T, C] -------------------
constexpr int kBnRows = 32;       // rows per partial: one 32-row MFMA tile of the projection GEMM

struct BnFinalArgs {
  const float* part_mean;   // [strips][2r] (training)
  const float* part_m2;
  float* stats;             // [4][r]: mean_x, rstd_x, mean_y, rstd_y
  void* running_mean[2];    // [r] each, dtype stat_dt; read in eval, updated in training
  void* running_var[2];
  int64_t* num_batches_tracked[2];   // may be NULL; read for the cumulative average (momentum < 0)
  int num_rows, r, strips, training, stat_dt;
  int count_here;                    // increment num_batches_tracked in this kernel (no select kernel follows; momentum >= 0 only)
  float momentum, eps;               // momentum < 0: cumulative moving average, factor 1 / (batches tracked so far + 1)
};

// One wave per column: merges the strip partials (mean = sum n_s mean_s / n,
// M2 = sum M2_s + n_s (mean_s - mean)^2, in double), writes mean and 1/sqrt(var+eps), and in
// training moves the running buffers (unbiased variance) as nn.BatchNorm1d does.  In eval
// the running buffers provide mean and variance.
__global__ __launch_bounds__(256) void bn_finalize_kernel(const BnFinalArgs g) {
  const int col = blockIdx.x * (256 / kWave) + (threadIdx.x >> 6), lane = lane_id();
  if (col == 0 && lane == 0 && g.training && g.count_here) {
    if (g.num_batches_tracked[0]) *g.num_batches_tracked[0] += 1;
    if (g.num_batches_tracked[1]) *g.num_batches_tracked[1] += 1;
  }
  if (col >= 2 * g.r) return;
  const int half = col >= g.r, key = col - half * g.r;
  float mean, var;
  if (g.training) {
    // the running buffers (and the batch count) are requested first: their latency passes beside the strips'
    const float rm = load_score(g.running_mean[half], key, g.stat_dt), rv = load_score(g.running_var[half], key, g.stat_dt);
    const float f = g.momentum >= 0.f ? g.momentum : 1.0f / (float)(*g.num_batches_tracked[half] + 1);
    // one pass over the strips, both sums in double: M2 = sum (M2_s + n_s mean_s^2) - n mu^2 (double carries 29 bits more than
    // the fp32 result keeps, so the difference stays exact to fp32 while mean^2 / variance < 2^29)
    double wsum = 0., q = 0.;
    for (int s = lane; s < g.strips; s += kWave) {
      const double ns = (double)min(kBnRows, g.num_rows - s * kBnRows), ms = (double)g.part_mean[int64_t(s) * 2 * g.r + col];
      wsum += ns * ms;
      q += (double)g.part_m2[int64_t(s) * 2 * g.r + col] + ns * ms * ms;
    }
    double sum2[2] = {wsum, q};
#pragma unroll
    for (int m = kWave / 2; m >= 1; m >>= 1) {
      const double o0 = __shfl_xor(sum2[0], m, kWave), o1 = __shfl_xor(sum2[1], m, kWave);
      sum2[0] += o0;
      sum2[1] += o1;
    }
    const double n = (double)g.num_rows, mu = sum2[0] / n;
    const double m2 = fmax(sum2[1] - n * mu * mu, 0.);
    mean = (float)mu;
    var = (float)(m2 / n);                                   // biased: normalises the batch
    if (lane == 0) {
      const float unbiased = (float)(m2 / (n > 1. ? n - 1. : 1.));
      // nn.BatchNorm1d(momentum=None): the factor f is 1 / num_batches_tracked AFTER this batch has been counted
      store_score(g.running_mean[half], key, (1.f - f) * rm + f * mean, g.stat_dt);
      store_score(g.running_var[half], key, (1.f - f) * rv + f * unbiased, g.stat_dt);
    }
  } else {
    mean = load_score(g.running_mean[half], key, g.stat_dt);
    var = load_score(g.running_var[half], key, g.stat_dt);
  }
  if (lane == 0) {
    g.stats[(2 * half) * g.r + key] = mean;
    g.stats[(2 * half + 1) * g.r + key] = 1.0f / sqrtf(var + g.eps);
  }
}

static inline size_t align256(size_t v) { return (v + 255) / 256 * 256; }

}  // namespace omni

extern "C" OMNI_API int32_t omni_router_select(const void* logits_x, const void* logits_y, void* scores, int32_t* indices,
                                               int64_t num_tokens, int32_t num_expert_sqrt, int32_t num_experts_per_token,
                                               int32_t dtype, void* stream) {
  using namespace omni;
  const int r = num_expert_sqrt, k = num_experts_per_token;
  if (num_tokens < 0 || num_tokens > INT32_MAX / 256 || r <= 0) return OMNI_ERR_SHAPE;
  if (k < 0 || (int64_t)k > (int64_t)r * r || k > 128 || (k & 1)) return OMNI_ERR_TOPK;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  if (num_tokens == 0 || k == 0) return OMNI_OK;
  if (!logits_x || !logits_y || !scores || !indices) return OMNI_ERR_NULL;
  if (!select_covers(r, k, dtype)) return OMNI_ERR_UNSUPPORTED;
  SelectArgs g{};
  g.lx = logits_x; g.ly = logits_y; g.row_stride = r; g.scores = scores; g.indices = indices;
  g.num_tokens = (int)num_tokens; g.r = r; g.k = k; g.dt = dtype;
  return select_dispatch(g, (hipStream_t)stream);
}

// workspace layout of omni_router_fwd: z [T,2r] | stats [4r] f32 | part_mean | part_m2
extern "C" OMNI_API size_t omni_router_workspace_bytes(int64_t num_tokens, int32_t num_expert_sqrt, int32_t dtype) {
  using namespace omni;
  if (num_tokens < 0 || num_expert_sqrt <= 0) return 0;
  const size_t es = dtype == OMNI_F32 ? 4 : 2, r = (size_t)num_expert_sqrt;
  const size_t strips = ((size_t)num_tokens + kBnRows - 1) / kBnRows;
  return align256((size_t)num_tokens * 2 * r * es) + align256(4 * r * 4) + 2 * align256(strips * 2 * r * 4);
}

// After omni_router_fwd the workspace still holds what a backward pass needs: z at offset 0 and,
// at this offset, the fp32 statistics [mean_x | rstd_x | mean_y | rstd_y], r values each.
extern "C" OMNI_API size_t omni_router_workspace_stats_offset(int64_t num_tokens, int32_t num_expert_sqrt, int32_t dtype) {
  using namespace omni;
  if (num_tokens < 0 || num_expert_sqrt <= 0) return 0;
  const size_t es = dtype == OMNI_F32 ? 4 : 2;
  return align256((size_t)num_tokens * 2 * (size_t)num_expert_sqrt * es);
}

extern "C" OMNI_API int32_t omni_router_fwd(const void* x, const void* weight_x, const void* weight_y,
                                            void* running_mean_x, void* running_var_x, int64_t* num_batches_tracked_x,
                                            void* running_mean_y, void* running_var_y, int64_t* num_batches_tracked_y,
                                            int32_t training, float momentum, float eps, void* gates, int32_t* indices,
                                            void* scores, int64_t num_tokens, int32_t hidden_size, int32_t num_expert_sqrt,
                                            int32_t num_experts_per_token, int32_t dtype, int32_t stats_dtype,
                                            void* workspace, void* stream) {
  using namespace omni;
  const int r = num_expert_sqrt, k = num_experts_per_token;
  if (num_tokens < 0 || num_tokens > INT32_MAX / 256 || r <= 0 || hidden_size <= 0) return OMNI_ERR_SHAPE;
  if (k < 0 || (int64_t)k > (int64_t)r * r || k > 128 || (k & 1)) return OMNI_ERR_TOPK;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  if (stats_dtype != OMNI_BF16 && stats_dtype != OMNI_F16 && stats_dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  if (num_tokens == 0) return OMNI_OK;
  if (training && num_tokens == 1) return OMNI_ERR_SHAPE;   // batch statistics of one sample: nn.BatchNorm1d raises
  if (!x || !weight_x || !weight_y || !running_mean_x || !running_var_x || !running_mean_y || !running_var_y) return OMNI_ERR_NULL;
  if (training && momentum < 0.f && (!num_batches_tracked_x || !num_batches_tracked_y)) return OMNI_ERR_NULL;   // the cumulative average needs the counts
  if (training && momentum < 0.f && k == 0) return OMNI_ERR_UNSUPPORTED;
  if (k > 0 && !select_covers(r, k, dtype)) return OMNI_ERR_UNSUPPORTED;   // the select kernels' limit, checked before the projection is enqueued
  if (k > 0 && (!gates || !indices)) return OMNI_ERR_NULL;
  if (!workspace) return OMNI_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  const size_t strips = ((size_t)num_tokens + kBnRows - 1) / kBnRows;
  char* w = (char*)workspace;
  const size_t es = dtype == OMNI_F32 ? 4 : 2;
  void* z = w;                       w += align256((size_t)num_tokens * 2 * r * es);
  float* stats = (float*)w;          w += align256((size_t)4 * r * 4);
  float* part_mean = (float*)w;      w += align256(strips * 2 * r * 4);
  float* part_m2 = (float*)w;

  // z = x [Wx;Wy]^T on the matrix cores
  // (in training its epilogue also leaves the per-32-row column statistics)
  if (int e = omni_gemm_router_projection(x, weight_x, weight_y, z, training ? part_mean : nullptr, training ? part_m2 : nullptr,
                                          num_tokens, hidden_size, r, dtype, stream)) return e;
  // Training: one more launch merges the partial statistics and moves the running buffers.  In eval mode the
  // select kernel reads the running buffers itself (and leaves mean and 1/sqrt(var + eps) in `stats`).
  if (training || k == 0) {
    BnFinalArgs b{part_mean, part_m2, stats, {running_mean_x, running_mean_y}, {running_var_x, running_var_y},
                  {num_batches_tracked_x, num_batches_tracked_y}, (int)num_tokens, r, (int)strips, training ? 1 : 0, stats_dtype,
                  k == 0 ? 1 : 0, momentum, eps};
    hipLaunchKernelGGL(bn_finalize_kernel, dim3((2 * r + 3) / 4), dim3(256), 0, s, b);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return OMNI_ERR_HIP_BASE + (int)err;
    if (k == 0) return OMNI_OK;
  }
  SelectArgs g{};
  g.lx = z; g.ly = (const char*)z + (size_t)r * es; g.row_stride = 2 * r;
  g.scores = scores; g.gates = gates; g.indices = indices;
  g.num_tokens = (int)num_tokens; g.r = r; g.k = k; g.dt = dtype;
  if (training) {
    g.stats = stats;
    g.count_batch[0] = num_batches_tracked_x; g.count_batch[1] = num_batches_tracked_y;
  } else {
    g.run_mean[0] = running_mean_x; g.run_mean[1] = running_mean_y;
    g.run_var[0] = running_var_x; g.run_var[1] = running_var_y;
    g.stats_out = stats; g.stat_dt = stats_dtype; g.eps = eps;
  }
  return select_dispatch(g, s);
}
