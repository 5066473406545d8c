// Fused atomic-expert forward for gfx950:
//     y[t,:] = sum_j silu(<x[t,:], U[id[t,j],:]>) * g[t,j] * V[id[t,j],:]
// replacing the reference's schedule + two Triton kernels + fp32 score buffer
// (omni_moe/ops/triton/omni_expert.py:8-168, 920-992) with one launch.
//
// Token-resident gather ("gather" algorithm): one 64-lane wave owns one token.
// The token's row of x stays in registers (16 B per lane per 1 KiB of row), each
// selected expert's up row and down row is fetched with one fully coalesced
// 128-bit load per lane per 1 KiB, the dot product is reduced across the wave,
// and the gate-weighted down rows accumulate in fp32 registers.  Nothing but y
// is written: no score buffer, no atomics, and the summation order is fixed
// (slot 0..k-1), so results are run-to-run identical.
//
// Expert-centric variant ("segment" algorithm), the reference's own organisation
// (omni_expert.py:8-168): the pairs are first grouped by expert (omni_schedule), then
//   A. waves walk the sorted pair list, 16 consecutive pairs each -- so a popular expert's
//      segment is spread over many waves and an unpopular one costs one short visit -- gather
//      the pair's x row and its expert's up row (which repeats along a segment and therefore
//      hits in cache), and write the coefficient silu(<x,u>)*g of the pair;
//   B. a token-resident pass accumulates coefficient * down row into y, in slot order.
// No atomics, same fixed summation order as the gather algorithm, hence identical results;
// it moves the same rows plus the schedule and a [T,k] fp32 coefficient buffer, and exists so
// that the two organisations can be measured side by side.
#include "common.h"
#include "omni_moe_hip.h"
#include "rows.h"

// gemm.hip: c[T, 2N] = [round(v) | round(v - round(v))], v = silu(x W^T) * gate
int omni_gemm_gated(const void* x, const void* w, const float* gate, void* c, int64_t T, int64_t N, int64_t K, int dtype, void* stream);

namespace omni {

constexpr int kTokensPerBlock = 4;   // one wave each

// NCH = 16-byte chunks of a row per lane (row bytes / 1024, rounded up);
// G   = experts fetched per batch (their 2*G*NCH loads are all in flight at once).
template <int DT, int NCH, int G>
__global__ __launch_bounds__(kTokensPerBlock* kWave, 2) void expert_gather_kernel(
    const uint8_t* __restrict__ x, const uint8_t* __restrict__ up, const uint8_t* __restrict__ down,
    const void* __restrict__ gates, const int32_t* __restrict__ ids, uint8_t* __restrict__ y,
    int num_tokens, int hidden, int top_k, uint32_t num_experts) {
  constexpr int E = Row16<DT>::kElems;
  const int lane = lane_id();
  const int t = __builtin_amdgcn_readfirstlane(blockIdx.x * kTokensPerBlock + (threadIdx.x >> 6));
  if (t >= num_tokens) return;
  const int64_t row_bytes = int64_t(hidden) * (16 / E);

  bool live[NCH];
  int64_t off[NCH];                    // byte offset of this lane's chunk c inside a row
  u32x4_t xr[NCH];
  float acc[NCH][E];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int first = (c * kWave + lane) * E;
    live[c] = first < hidden;
    off[c] = int64_t(c * kWave + lane) * 16;
    xr[c] = live[c] ? *(const u32x4_t*)(x + t * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < E; ++i) acc[c][i] = 0.f;
  }

  const int32_t* my_ids = ids + int64_t(t) * top_k;
  for (int j0 = 0; j0 < top_k; j0 += G) {
    int e[G];
    float g[G];
    bool live_slot[G];
#pragma unroll
    for (int i = 0; i < G; ++i) {
      const int j = min(j0 + i, top_k - 1);          // always a valid slot: no branch around the loads
      const int id = my_ids[j];
      const float gate = Elem<DT>::load(gates, int64_t(t) * top_k + j);
      // a slot past k, or an id outside the table, contributes nothing
      const bool ok = (j0 + i < top_k) && (uint32_t)id < num_experts;
      e[i] = ok ? id : 0;
      g[i] = ok ? gate : 0.f;
      live_slot[i] = ok;
    }
    u32x4_t ur[G][NCH], vr[G][NCH];
#pragma unroll
    for (int i = 0; i < G; ++i)
#pragma unroll
      for (int c = 0; c < NCH; ++c)
        ur[i][c] = live[c] ? *(const u32x4_t*)(up + e[i] * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < G; ++i)
#pragma unroll
      for (int c = 0; c < NCH; ++c)
        vr[i][c] = live[c] ? *(const u32x4_t*)(down + e[i] * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};

    float s[G];
#pragma unroll
    for (int i = 0; i < G; ++i) {
      float p = 0.f;
#pragma unroll
      for (int c = 0; c < NCH; ++c) p = dot16<DT>(xr[c], ur[i][c], p);
      s[i] = p;
    }
#pragma unroll
    for (int i = 0; i < G; ++i) s[i] = wave_sum(s[i]);
#pragma unroll
    for (int i = 0; i < G; ++i) {
      if (!live_slot[i]) continue;                  // not even 0 * row: the stand-in row may hold Inf or NaN
      const float coef = silu_f32(s[i]) * g[i];
#pragma unroll
      for (int c = 0; c < NCH; ++c) axpy16<DT>(coef, vr[i][c], acc[c]);
    }
  }

#pragma unroll
  for (int c = 0; c < NCH; ++c)
    if (live[c]) *(u32x4_t*)(y + t * row_bytes + off[c]) = pack16<DT>(acc[c]);
}

template <int DT, int NCH, int G>
static hipError_t launch_gather(const void* x, const void* up, const void* down, const void* gates,
                                const int32_t* ids, void* y, int64_t T, int H, int k, int64_t N, hipStream_t s) {
  if (T == 0) return hipSuccess;
  dim3 grid((unsigned)((T + kTokensPerBlock - 1) / kTokensPerBlock)), block(kTokensPerBlock * kWave);
  hipLaunchKernelGGL((expert_gather_kernel<DT, NCH, G>), grid, block, 0, s, (const uint8_t*)x, (const uint8_t*)up,
                     (const uint8_t*)down, gates, ids, (uint8_t*)y, (int)T, H, k, (uint32_t)N);
  return hipGetLastError();
}

template <int DT>
static int expert_gather_dispatch(const void* x, const void* up, const void* down, const void* gates,
                                  const int32_t* ids, void* y, int64_t T, int H, int k, int64_t N, hipStream_t s) {
  constexpr int E = Row16<DT>::kElems;
  if (H % E != 0) return OMNI_ERR_SHAPE;              // rows must be 16-byte multiples
  const int nch = (H + kWave * E - 1) / (kWave * E);
  hipError_t err;
  if (nch <= 1) err = launch_gather<DT, 1, 16>(x, up, down, gates, ids, y, T, H, k, N, s);
  else if (nch <= 2) err = launch_gather<DT, 2, 8>(x, up, down, gates, ids, y, T, H, k, N, s);
  else if (nch <= 4) err = launch_gather<DT, 4, 4>(x, up, down, gates, ids, y, T, H, k, N, s);
  else if (nch <= 8) err = launch_gather<DT, 8, 2>(x, up, down, gates, ids, y, T, H, k, N, s);
  else return OMNI_ERR_UNSUPPORTED;
  return err == hipSuccess ? OMNI_OK : OMNI_ERR_HIP_BASE + (int)err;
}

// ---- expert-centric variant -------------------------------------------------------------------
constexpr int kPairsPerWave = 16;

template <int DT, int NCH>
__global__ __launch_bounds__(256, 2) void expert_segment_scores_kernel(
    const uint8_t* __restrict__ x, const uint8_t* __restrict__ up, const void* __restrict__ gates,
    const int32_t* __restrict__ ids, const int32_t* __restrict__ sorted_pair_ids, const int32_t* __restrict__ offsets,
    float* __restrict__ coef, int hidden, int top_k, int64_t num_experts) {
  constexpr int E = Row16<DT>::kElems;
  constexpr int G = (NCH <= 2) ? 8 : (NCH <= 4 ? 4 : 2);       // pairs whose rows are in flight together
  const int lane = lane_id();
  const int num_valid = offsets[num_experts];                   // pairs with an id inside the table
  const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
  const int pos0 = wave * kPairsPerWave;
  if (pos0 >= num_valid) return;
  const int64_t row_bytes = int64_t(hidden) * (16 / E);
  bool live[NCH];
  int64_t off[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    live[c] = (c * kWave + lane) * E < hidden;
    off[c] = int64_t(c * kWave + lane) * 16;
  }
  for (int g0 = 0; g0 < kPairsPerWave; g0 += G) {
    int pid[G];
    bool ok[G];
    u32x4_t xr[G][NCH], ur[G][NCH];
#pragma unroll
    for (int i = 0; i < G; ++i) {
      const int pos = pos0 + g0 + i;
      ok[i] = pos < num_valid;
      pid[i] = sorted_pair_ids[ok[i] ? pos : pos0];
      const int t = pid[i] / top_k, e = ids[pid[i]];
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        xr[i][c] = live[c] ? *(const u32x4_t*)(x + t * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};
        ur[i][c] = live[c] ? *(const u32x4_t*)(up + e * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};
      }
    }
#pragma unroll
    for (int i = 0; i < G; ++i) {
      float p = 0.f;
#pragma unroll
      for (int c = 0; c < NCH; ++c) p = dot16<DT>(xr[i][c], ur[i][c], p);
      const float sdot = wave_sum(p);
      if (ok[i] && lane == 0) coef[pid[i]] = silu_f32(sdot) * Elem<DT>::load(gates, pid[i]);
    }
  }
}

// y[t] = sum_j coef[t,j] * down[id[t,j]] in slot order; coef comes from the scores pass.
template <int DT, int NCH, int G>
__global__ __launch_bounds__(kTokensPerBlock* kWave, 2) void expert_accumulate_kernel(
    const uint8_t* __restrict__ down, const float* __restrict__ coef, const int32_t* __restrict__ ids,
    uint8_t* __restrict__ y, int num_tokens, int hidden, int top_k, uint32_t num_experts) {
  constexpr int E = Row16<DT>::kElems;
  const int lane = lane_id();
  const int t = __builtin_amdgcn_readfirstlane(blockIdx.x * kTokensPerBlock + (threadIdx.x >> 6));
  if (t >= num_tokens) return;
  const int64_t row_bytes = int64_t(hidden) * (16 / E);
  bool live[NCH];
  int64_t off[NCH];
  float acc[NCH][E];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    live[c] = (c * kWave + lane) * E < hidden;
    off[c] = int64_t(c * kWave + lane) * 16;
#pragma unroll
    for (int i = 0; i < E; ++i) acc[c][i] = 0.f;
  }
  for (int j0 = 0; j0 < top_k; j0 += G) {
    float cf[G];
    bool used[G];
    u32x4_t vr[G][NCH];
#pragma unroll
    for (int i = 0; i < G; ++i) {
      const int j = min(j0 + i, top_k - 1);
      const int id = ids[int64_t(t) * top_k + j];
      const bool ok = (j0 + i < top_k) && (uint32_t)id < num_experts;
      used[i] = ok;
      cf[i] = ok ? coef[int64_t(t) * top_k + j] : 0.f;
      const int e = ok ? id : 0;
#pragma unroll
      for (int c = 0; c < NCH; ++c)
        vr[i][c] = live[c] ? *(const u32x4_t*)(down + e * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < G; ++i) {
      if (!used[i]) continue;
#pragma unroll
      for (int c = 0; c < NCH; ++c) axpy16<DT>(cf[i], vr[i][c], acc[c]);
    }
  }
#pragma unroll
  for (int c = 0; c < NCH; ++c)
    if (live[c]) *(u32x4_t*)(y + t * row_bytes + off[c]) = pack16<DT>(acc[c]);
}

static inline size_t align256(size_t v) { return (v + 255) / 256 * 256; }

template <int DT, int NCH, int G>
static hipError_t launch_segment(const void* x, const void* up, const void* down, const void* gates, const int32_t* ids,
                                 const int32_t* sorted_pair_ids, const int32_t* offsets, float* coef, void* y, int64_t T,
                                 int H, int k, int64_t N, hipStream_t s) {
  const int64_t P = T * k;
  const unsigned waves = (unsigned)((P + kPairsPerWave - 1) / kPairsPerWave);
  hipLaunchKernelGGL((expert_segment_scores_kernel<DT, NCH>), dim3((waves + 3) / 4), dim3(256), 0, s, (const uint8_t*)x,
                     (const uint8_t*)up, gates, ids, sorted_pair_ids, offsets, coef, H, k, N);
  hipLaunchKernelGGL((expert_accumulate_kernel<DT, NCH, G>), dim3((unsigned)((T + kTokensPerBlock - 1) / kTokensPerBlock)),
                     dim3(kTokensPerBlock * kWave), 0, s, (const uint8_t*)down, coef, ids, (uint8_t*)y, (int)T, H, k, (uint32_t)N);
  return hipGetLastError();
}

// workspace: offsets [N+1] | sorted pair ids [P] | coefficients [P] f32 | schedule workspace
template <int DT>
static int expert_segment_dispatch(const void* x, const void* up, const void* down, const void* gates, const int32_t* ids,
                                   void* y, int64_t T, int H, int k, int64_t N, void* workspace, hipStream_t s) {
  constexpr int E = Row16<DT>::kElems;
  if (H % E != 0) return OMNI_ERR_SHAPE;
  if (T == 0) return OMNI_OK;
  if (k == 0) return expert_gather_dispatch<DT>(x, up, down, gates, ids, y, T, H, k, N, s);   // writes zeros
  if (!workspace) return OMNI_ERR_WORKSPACE;
  const int64_t P = T * k;
  char* w = (char*)workspace;
  int32_t* offsets = (int32_t*)w;          w += align256((size_t)(N + 1) * 4);
  int32_t* sorted_pair_ids = (int32_t*)w;  w += align256((size_t)P * 4);
  float* coef = (float*)w;                 w += align256((size_t)P * 4);
  if (int e = omni_schedule(ids, offsets, sorted_pair_ids, nullptr, T, k, N, w, s)) return e;
  const int nch = (H + kWave * E - 1) / (kWave * E);
  hipError_t err;
  if (nch <= 1) err = launch_segment<DT, 1, 16>(x, up, down, gates, ids, sorted_pair_ids, offsets, coef, y, T, H, k, N, s);
  else if (nch <= 2) err = launch_segment<DT, 2, 8>(x, up, down, gates, ids, sorted_pair_ids, offsets, coef, y, T, H, k, N, s);
  else if (nch <= 4) err = launch_segment<DT, 4, 4>(x, up, down, gates, ids, sorted_pair_ids, offsets, coef, y, T, H, k, N, s);
  else if (nch <= 8) err = launch_segment<DT, 8, 2>(x, up, down, gates, ids, sorted_pair_ids, offsets, coef, y, T, H, k, N, s);
  else return OMNI_ERR_UNSUPPORTED;
  return err == hipSuccess ? OMNI_OK : OMNI_ERR_HIP_BASE + (int)err;
}

// ---- hidden-split variant ("split" algorithm) ------------------------------------------------
// For tables that fit the chip's caches but not one XCD's 4 MiB L2 (16 MiB at N = 4096,
// H = 1024): the hidden dimension is cut into 8 slices and slice s is only ever touched by
// blocks with blockIdx % 8 == s, which the dispatcher places on XCD s.  An XCD then needs
// N * H/8 elements of each table -- 1 MiB each in that example -- and serves every table row
// from its own L2 instead of pulling three quarters of them over the fabric.  The price is a
// cross-slice reduction of the pair scores, which is tiny ([8][T][k] floats):
//   A. block (token group, slice): partial dot products <x[t, slice], up[id, slice]> for the k pairs
//      of each of its tokens -> partial[slice][t][j];
//   B. block (token group, slice): coefficient silu(sum over slices, in slice order) * gate, then
//      y[t, slice] = sum_j coefficient_j * down[id_j, slice].
// A row slice is LPR lanes of 16 bytes (64 / LPR pairs per wave at a time).  Fixed summation
// order, no atomics; results agree with the gather algorithm to fp32 rounding of the dot product.
constexpr int kSlices = 8;

// Sum over the LPR lanes of a group of LPR values per lane, scattered: lane `sub` of the group
// ends up with the total of value `sub`.  Every step halves what a lane keeps (LPR - 1 exchanges
// in all, against LPR * log2(LPR) for one tree per value).
template <int LPR, int N = LPR>
__device__ __forceinline__ float reduce_scatter_group(float (&v)[N], const int lane) {
  if constexpr (N == 1) {
    return v[0];
  } else {
    constexpr int S = N / 2;                   // lane distance of this step = half of what is left
    const bool upper = lane & S;
    float keep[S];
#pragma unroll
    for (int e = 0; e < S; ++e) keep[e] = (upper ? v[e + S] : v[e]) + xor_lane_f<S>(upper ? v[e] : v[e + S], lane);
    return reduce_scatter_group<LPR, S>(keep, lane);
  }
}

// A wave owns GP = 64 / LPR tokens, one per lane group; the group's LPR lanes cover the token's
// row slice, 16 bytes each.  Pairs go in batches of LPR: LPR partial dot products per lane,
// then one reduce-scatter leaves pair `sub` of the batch in lane `sub`.
// SMALL: every table, x, y and the partial sums stay below 4 GiB, ids and row lengths below 2^24 (split_offsets_small):
// a row's byte offset is then one full-rate v_mad_u32_u24 on 32-bit lane offsets instead of a 64-bit multiply-add and two
// 32-bit multiplies at a quarter of the rate -- address arithmetic was more than half of the vector instructions' time here.
template <bool SMALL> struct SplitOff { using type = int64_t; };
template <> struct SplitOff<true> { using type = uint32_t; };
template <bool SMALL>
__device__ __forceinline__ typename SplitOff<SMALL>::type split_mul(uint32_t a, typename SplitOff<SMALL>::type b) {
  if constexpr (SMALL) return __umul24(a, b); else return (int64_t)a * b;
}

template <int DT, int LPR, bool SMALL>
__global__ __launch_bounds__(kTokensPerBlock* kWave) void expert_split_dots_kernel(
    const uint8_t* __restrict__ x, const uint8_t* __restrict__ up, const int32_t* __restrict__ ids,
    float* __restrict__ partial, int num_tokens, int hidden, int top_k, uint32_t num_experts, int col_block) {
  using Off = typename SplitOff<SMALL>::type;
  constexpr int E = Row16<DT>::kElems, GP = kWave / LPR;
  constexpr int LD = LPR < 8 ? LPR : 8;                          // row loads in flight at a time
  const int lane = lane_id(), sub = lane % LPR, grp = lane / LPR;
  const int slice = blockIdx.x % kSlices;
  const int t = ((int)(blockIdx.x / kSlices) * kTokensPerBlock + (threadIdx.x >> 6)) * GP + grp;
  const bool live = t < num_tokens;
  const int tt = live ? t : 0;
  const Off row_bytes = Off(hidden) * (16 / E);
  // this lane's 16 bytes inside a row (rows wider than 8 slices of 64 lanes go in column blocks of 8 slices, one launch each)
  const Off col = (Off(col_block) * kSlices + slice) * LPR * 16 + sub * 16;
  const u32x4_t xr = *(const u32x4_t*)(x + (split_mul<SMALL>((uint32_t)tt, row_bytes) + col));
  const Off base = split_mul<SMALL>((uint32_t)tt, (Off)top_k);
  for (int jb = 0; jb < top_k; jb += LPR) {
    // lane `sub` of a group fetches the id of pair `sub` of the batch; the group reads the ids from its lanes
    const int my_id = ids[base + min(jb + sub, top_k - 1)];
    float d[LPR];
#pragma unroll
    for (int e0 = 0; e0 < LPR; e0 += LD) {
      u32x4_t ur[LD];
#pragma unroll
      for (int e = 0; e < LD; ++e) {
        const int id = __shfl(my_id, grp * LPR + e0 + e, kWave);
        ur[e] = *(const u32x4_t*)(up + (split_mul<SMALL>((uint32_t)id < num_experts ? (uint32_t)id : 0u, row_bytes) + col));
      }
#pragma unroll
      for (int e = 0; e < LD; ++e) d[e0 + e] = dot16<DT>(xr, ur[e], 0.f);
    }
    const float total = reduce_scatter_group<LPR>(d, lane);
    const int j = jb + sub;
    if (live && j < top_k) {
      const bool ok = (uint32_t)my_id < num_experts;
      partial[((Off(col_block) * kSlices + slice) * num_tokens + t) * top_k + j] = ok ? total : 0.f;
    }
  }
}

// Same ownership.  Lane `sub` of a group forms the coefficient of pair `sub` of a batch (sum of
// the 8 slice partials in slice order, silu, gate); the group then walks the batch, every lane
// fetching its 16 bytes of the down row and the pair's coefficient from the lane that holds it.
// WIDE: rows of several column blocks (col_block of col_blocks); otherwise both are compile-time constants, which keeps
// the eight partial-sum loads of the common case one unrolled group that the compiler places behind the row requests.
template <int DT, int LPR, bool WIDE, bool SMALL>
__global__ __launch_bounds__(kTokensPerBlock* kWave) void expert_split_accumulate_kernel(
    const uint8_t* __restrict__ down, const void* __restrict__ gates, const int32_t* __restrict__ ids,
    const float* __restrict__ partial, uint8_t* __restrict__ y, int num_tokens, int hidden, int top_k, uint32_t num_experts,
    int col_block_arg, int col_blocks_arg) {
  using Off = typename SplitOff<SMALL>::type;
  const int col_block = WIDE ? col_block_arg : 0, col_blocks = WIDE ? col_blocks_arg : 1;
  constexpr int E = Row16<DT>::kElems, GP = kWave / LPR;
  constexpr int LD = LPR < 8 ? LPR : 8;
  const int lane = lane_id(), sub = lane % LPR, grp = lane / LPR;
  const int slice = blockIdx.x % kSlices;
  const int t = ((int)(blockIdx.x / kSlices) * kTokensPerBlock + (threadIdx.x >> 6)) * GP + grp;
  const bool live = t < num_tokens;
  const int tt = live ? t : 0;
  const Off row_bytes = Off(hidden) * (16 / E);
  const Off col = (Off(col_block) * kSlices + slice) * LPR * 16 + sub * 16;
  const Off base = split_mul<SMALL>((uint32_t)tt, (Off)top_k);
  float acc[E];
#pragma unroll
  for (int i = 0; i < E; ++i) acc[i] = 0.f;
  for (int jb = 0; jb < top_k; jb += LPR) {
    const int j = jb + sub;
    int my_id = -1;                                               // -1: a padded slot or an id outside the table
    if (j < top_k) {
      const int id = ids[base + j];
      if ((uint32_t)id < num_experts) my_id = id;
    }
    // the down rows only need the ids: the first LD of them are requested ahead of the partial sums the coefficients
    // wait for; every row that has been added makes room for the request of a later one (LD row registers in all)
    u32x4_t vr[LD];
    bool used[LD];
    auto request = [&](int slot, int e) {
      const int id = __shfl(my_id, grp * LPR + e, kWave);         // from the lane of this group that holds pair e
      used[slot] = id >= 0;
      vr[slot] = *(const u32x4_t*)(down + (split_mul<SMALL>(used[slot] ? (uint32_t)id : 0u, row_bytes) + col));
    };
#pragma unroll
    for (int e = 0; e < LD; ++e) request(e, e);
    float coef = 0.f;
    if (my_id >= 0) {
      float sdot = 0.f;
      for (int cb = 0; cb < col_blocks; ++cb) {                  // slice order, column block by column block
#pragma unroll
        for (int sl = 0; sl < kSlices; ++sl) sdot += partial[((Off(cb) * kSlices + sl) * num_tokens + tt) * top_k + j];
      }
      coef = silu_f32(sdot) * Elem<DT>::load(gates, base + j);
    }
#pragma unroll
    for (int e = 0; e < LPR; ++e) {
      const float cf = __shfl(coef, grp * LPR + e, kWave);
      if (used[e % LD]) axpy16<DT>(cf, vr[e % LD], acc);          // not even 0 * row: the stand-in row may hold Inf or NaN
      if (e + LD < LPR) request(e % LD, e + LD);
    }
  }
  if (live) *(u32x4_t*)(y + (split_mul<SMALL>((uint32_t)t, row_bytes) + col)) = pack16<DT>(acc);
}

// lanes per row slice, or 0 when the row does not cut into 8 slices of 4..64 lanes
static inline int split_lanes_per_row(int hidden, int elem_bytes) {
  const int64_t slice_bytes = (int64_t)hidden * elem_bytes / kSlices;
  if ((int64_t)hidden * elem_bytes % (kSlices * 16) != 0) return 0;
  const int lpr = (int)(slice_bytes / 16);
  return (lpr == 4 || lpr == 8 || lpr == 16 || lpr == 32 || lpr == 64) ? lpr : 0;
}
// Rows beyond 8 KiB (8 slices of 64 lanes): the smallest number of column blocks, each 8 slices of a power-of-two number of
// lanes, that the row cuts into; 0 if there is none (up to 64 blocks: rows of 512 KiB).  1 for rows that split_lanes_per_row takes.
constexpr int kMaxColBlocks = 64;
static inline int split_col_blocks(int hidden, int elem_bytes, int* lanes_per_row) {
  for (int b = 1; b <= kMaxColBlocks; ++b) {
    if (hidden % b != 0) continue;
    const int lpr = split_lanes_per_row(hidden / b, elem_bytes);
    if (lpr) { *lanes_per_row = lpr; return b; }
  }
  return 0;
}

// every byte offset into x, y, the tables and the partial sums fits 32 bits, and the factors of its products 24
static inline bool split_offsets_small(int64_t T, int H, int k, int64_t N, int col_blocks, int elem_bytes) {
  const int64_t row = (int64_t)H * elem_bytes, lim = (int64_t)1 << 32, f24 = (int64_t)1 << 24;
  return row < f24 && N < f24 && T < f24 && k < f24 && N * row < lim && T * row < lim && T * k < lim &&
         (int64_t)kSlices * col_blocks * T * k * 4 < lim;
}

template <int DT, int LPR, bool SMALL>
static hipError_t launch_split_as(const void* x, const void* up, const void* down, const void* gates, const int32_t* ids,
                                  float* partial, void* y, int64_t T, int H, int k, int64_t N, int col_blocks, hipStream_t s) {
  constexpr int kPerBlock = kTokensPerBlock * (kWave / LPR);       // tokens per block
  // measured (bf16, same box): the dots pass gains 1-3 % from 32-bit offsets at every slice length; the accumulate pass gains
  // 3 % at 512-byte slices and LOSES 4-8 % at 256-byte ones (the compiler's schedule of its row window changes with them)
  constexpr bool kAccSmall = SMALL && LPR >= 32;
  const unsigned blocks = (unsigned)((T + kPerBlock - 1) / kPerBlock) * kSlices;
  for (int cb = 0; cb < col_blocks; ++cb)                            // all partial dot products first: a coefficient needs the whole row
    hipLaunchKernelGGL((expert_split_dots_kernel<DT, LPR, SMALL>), dim3(blocks), dim3(kTokensPerBlock * kWave), 0, s, (const uint8_t*)x,
                       (const uint8_t*)up, ids, partial, (int)T, H, k, (uint32_t)N, cb);
  if (col_blocks == 1) {
    hipLaunchKernelGGL((expert_split_accumulate_kernel<DT, LPR, false, kAccSmall>), dim3(blocks), dim3(kTokensPerBlock * kWave), 0, s,
                       (const uint8_t*)down, gates, ids, partial, (uint8_t*)y, (int)T, H, k, (uint32_t)N, 0, 1);
    return hipGetLastError();
  }
  for (int cb = 0; cb < col_blocks; ++cb)
    hipLaunchKernelGGL((expert_split_accumulate_kernel<DT, LPR, true, kAccSmall>), dim3(blocks), dim3(kTokensPerBlock * kWave), 0, s,
                       (const uint8_t*)down, gates, ids, partial, (uint8_t*)y, (int)T, H, k, (uint32_t)N, cb, col_blocks);
  return hipGetLastError();
}
template <int DT, int LPR>
static hipError_t launch_split(const void* x, const void* up, const void* down, const void* gates, const int32_t* ids,
                               float* partial, void* y, int64_t T, int H, int k, int64_t N, int col_blocks, hipStream_t s) {
  if (split_offsets_small(T, H, k, N, col_blocks, DT == kF32 ? 4 : 2))
    return launch_split_as<DT, LPR, true>(x, up, down, gates, ids, partial, y, T, H, k, N, col_blocks, s);
  return launch_split_as<DT, LPR, false>(x, up, down, gates, ids, partial, y, T, H, k, N, col_blocks, s);
}

// workspace: partial dot products [8 * column blocks][T][k] f32
template <int DT>
static int expert_split_dispatch(const void* x, const void* up, const void* down, const void* gates, const int32_t* ids,
                                 void* y, int64_t T, int H, int k, int64_t N, void* workspace, hipStream_t s) {
  int lpr = 0;
  const int col_blocks = split_col_blocks(H, DT == kF32 ? 4 : 2, &lpr);
  if (col_blocks == 0 || k > 2 * kWave) return OMNI_ERR_UNSUPPORTED;
  if (T == 0) return OMNI_OK;
  if (k == 0) return expert_gather_dispatch<DT>(x, up, down, gates, ids, y, T, H, k, N, s);   // writes zeros
  if (!workspace) return OMNI_ERR_WORKSPACE;
  float* partial = (float*)workspace;
  hipError_t err;
  if (lpr == 4) err = launch_split<DT, 4>(x, up, down, gates, ids, partial, y, T, H, k, N, col_blocks, s);
  else if (lpr == 8) err = launch_split<DT, 8>(x, up, down, gates, ids, partial, y, T, H, k, N, col_blocks, s);
  else if (lpr == 16) err = launch_split<DT, 16>(x, up, down, gates, ids, partial, y, T, H, k, N, col_blocks, s);
  else if (lpr == 32) err = launch_split<DT, 32>(x, up, down, gates, ids, partial, y, T, H, k, N, col_blocks, s);
  else err = launch_split<DT, 64>(x, up, down, gates, ids, partial, y, T, H, k, N, col_blocks, s);
  return err == hipSuccess ? OMNI_OK : OMNI_ERR_HIP_BASE + (int)err;
}

// ---- dense variant ("dense" algorithm) --------------------------------------------------------
// The regime of the reference's group path (omni_scheduler.py:58,103-226; omni_expert.py:171-372): so few experts
// that each serves hundreds of tokens (T*k/N > 256).  The reference looks for 16 experts with identical token lists
// and runs those through tl.dot; here the whole op becomes two MFMA GEMMs over ALL experts, which at this density
// cost less than fetching 2k rows per token:
//   G[t, e]  = sum of the gates of token t's slots that name expert e (0 elsewhere)      gate matrix, fp32
//   C        = silu(x U^T) * G, kept as a 16-bit head and a 16-bit remainder [T, 2N]      GEMM with a gate epilogue
//   y        = [C_head | C_rem] [V^T | V^T]^T                                             GEMM over K = 2N
// silu and the gate product are fp32, C carries 16 significant bits, sums are fp32: results agree with the gather
// algorithm to a few units of fp32 rounding of the coefficients.  Duplicate slots add their gates in slot order.
constexpr int kDenseMaxExperts = 2048;

// One wave per token: the token's row of G is built in LDS (slots in order, by one lane) and written out whole.
__global__ __launch_bounds__(256) void dense_gate_rows_kernel(const void* __restrict__ gates, const int32_t* __restrict__ ids,
                                                              float* __restrict__ gate_matrix, int num_tokens, int top_k,
                                                              int num_experts, int dtype) {
  extern __shared__ float rows[];                                  // [4 waves][num_experts]
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  const int t = blockIdx.x * 4 + wave;
  if (t >= num_tokens) return;
  float* row = rows + wave * num_experts;
  for (int e = lane; e < num_experts; e += kWave) row[e] = 0.f;
  __builtin_amdgcn_wave_barrier();
  if (lane == 0) {
    for (int j = 0; j < top_k; ++j) {
      const int id = ids[(int64_t)t * top_k + j];
      if ((uint32_t)id < (uint32_t)num_experts) {
        const float g = dtype == OMNI_BF16 ? Elem<kBF16>::load(gates, (int64_t)t * top_k + j) : Elem<kF16>::load(gates, (int64_t)t * top_k + j);
        row[id] += g;
      }
    }
  }
  __builtin_amdgcn_wave_barrier();
  for (int e = lane; e < num_experts; e += kWave) gate_matrix[(int64_t)t * num_experts + e] = row[e];
}

// vt2[h, c] = v[c % N, h] for c < 2N: the down table transposed, twice side by side (K-contiguous operand of the second GEMM)
__global__ __launch_bounds__(256) void dense_transpose_kernel(const uint16_t* __restrict__ v, uint16_t* __restrict__ vt2, int num_experts, int hidden) {
  __shared__ uint16_t tile[64][66];
  const int e0 = blockIdx.x * 64, h0 = blockIdx.y * 64;
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    const int e = i / 64, h = i % 64;
    tile[e][h] = (e0 + e < num_experts && h0 + h < hidden) ? v[(int64_t)(e0 + e) * hidden + h0 + h] : (uint16_t)0;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    const int h = i / 64, e = i % 64;
    if (e0 + e < num_experts && h0 + h < hidden) {
      const uint16_t x = tile[e][h];
      vt2[(int64_t)(h0 + h) * 2 * num_experts + e0 + e] = x;
      vt2[(int64_t)(h0 + h) * 2 * num_experts + num_experts + e0 + e] = x;
    }
  }
}

static inline bool dense_covers(int64_t T, int H, int64_t N, int k, int dtype) {
  return dtype != OMNI_F32 && N % 32 == 0 && N <= kDenseMaxExperts && H % 64 == 0 && H % 8 == 0 && k > 0 && T > 0;
}

// workspace: gate matrix [T, N] f32 | coefficients [T, 2N] | transposed down table [H, 2N]
static inline size_t dense_workspace_bytes(int64_t T, int H, int64_t N) {
  return align256((size_t)T * N * 4) + align256((size_t)T * 2 * N * 2) + align256((size_t)H * 2 * N * 2);
}

static int expert_dense_dispatch(const void* x, const void* up, const void* down, const void* gates, const int32_t* ids, void* y,
                                 int64_t T, int H, int k, int64_t N, int dtype, void* workspace, hipStream_t s) {
  if (T == 0) return OMNI_OK;
  if (!dense_covers(T, H, N, k, dtype)) return OMNI_ERR_UNSUPPORTED;
  if (!workspace) return OMNI_ERR_WORKSPACE;
  char* w = (char*)workspace;
  float* gate_matrix = (float*)w;  w += align256((size_t)T * N * 4);
  void* coef = w;                  w += align256((size_t)T * 2 * N * 2);
  uint16_t* vt2 = (uint16_t*)w;
  hipLaunchKernelGGL(dense_gate_rows_kernel, dim3((unsigned)((T + 3) / 4)), dim3(256), (size_t)4 * N * 4, s, gates, ids, gate_matrix, (int)T, k, (int)N, dtype);
  hipLaunchKernelGGL(dense_transpose_kernel, dim3((unsigned)((N + 63) / 64), (unsigned)((H + 63) / 64)), dim3(256), 0, s,
                     (const uint16_t*)down, vt2, (int)N, H);
  if (hipError_t e = hipGetLastError(); e != hipSuccess) return OMNI_ERR_HIP_BASE + (int)e;
  if (int e = omni_gemm_gated(x, up, gate_matrix, coef, T, N, H, dtype, s)) return e;
  return omni_linear_fwd(coef, vt2, nullptr, y, T, (int32_t)(2 * N), H, dtype, s);
}

// What OMNI_EXPERT_ALGO_AUTO runs, from the sizes alone.  The split algorithm gives every XCD an eighth of each table row,
// so it pays while an XCD's share of the tables stays near its caches (its 4 MiB L2 and its part of the memory-side cache)
// and a row slice is long enough to fetch well; whole-row gathering wins on short rows, on tables far beyond the caches
// and with few pairs (the split algorithm's second launch: at 32768 pairs it wins from 512-byte slices on, or from 16 MiB
// of tables on with 256-byte slices).  Measured with ids uniform over the experts, bf16, 4096 /
// 16384 / 32768 tokens x 16 / 16 / 32 experts per token, time of split over time of gather:
//   slice  64 B (hidden  256): 1.3-3.4 at every table size                        -> gather
//   slice 128 B (hidden  512): 0.72-0.91 up to 32 MiB of tables from 262144 pairs on, 1.02-1.6 beyond
//   slice 256 B (hidden 1024): 0.49-0.67 up to 64 MiB, 0.95-1.01 at 256 MiB, 1.03-1.14 beyond
//   slice 512 B (hidden 2048): 0.37-0.77 up to 128 MiB, 0.9 at 256 MiB; beyond, 0.89-0.99 from 262144 pairs on and 1.04-1.16 with 65536
//   slice   1 KiB (hidden 4096): 0.59-0.95 with 32 experts per token (a token's pairs fill half of the 64 lanes that
//                                share out a batch), 1.05-1.38 with 16
// A skewed router (few live experts) moves every figure towards the split algorithm; the caller who knows says so.
static int resolve_algo(int algo, int64_t T, int H, int64_t N, int k, int dtype) {
  if (algo != OMNI_EXPERT_ALGO_AUTO) return algo;
  // The dense algorithm is never chosen here: it multiplies every token by every table row, so one non-finite value
  // in a row that nobody selected would reach every token (0 * Inf), where the other algorithms and the reference
  // only ever touch selected rows; and where it wins at all it wins little (the reference's group regime, T*k/N > 256
  // with N <= 16 k: 63 us against 67.5 us gather at 16384 tokens, hidden 1024, N = 256, k = 16; 95 against 70 at N = 512).
  const int es = dtype == OMNI_F32 ? 4 : 2;
  // rows beyond 8 KiB do not fit the gather kernel's registers: the split kernels take them in column blocks
  if ((int64_t)H * es > 8192) return OMNI_EXPERT_ALGO_SPLIT;
  const int64_t tables = 2 * N * (int64_t)H * es, pairs = T * (int64_t)k;
  const int lpr = split_lanes_per_row(H, es);           // 16-byte lanes per row slice: 4 .. 64, or 0
  if (lpr < 8 || k > 2 * kWave || tables <= (3ll << 20) || pairs < 32768) return OMNI_EXPERT_ALGO_GATHER;
  bool split;
  if (lpr == 8) split = tables <= (32ll << 20) && pairs >= 131072;
  else if (lpr == 16) split = tables <= (128ll << 20) && (pairs >= 65536 || tables >= (16ll << 20));
  else split = (tables <= (256ll << 20) || pairs >= 262144) && 2 * k >= lpr;
  return split ? OMNI_EXPERT_ALGO_SPLIT : OMNI_EXPERT_ALGO_GATHER;
}

// OMNI_OK when omni_expert_fwd takes `algo` for these sizes (what the whole-layer call checks before it enqueues anything).
int expert_algo_check(int algo, int64_t T, int H, int64_t N, int k, int dtype) {
  const int es = dtype == OMNI_F32 ? 4 : 2;
  switch (algo) {
    case OMNI_EXPERT_ALGO_AUTO:
      if ((int64_t)H * es <= 8192) return OMNI_OK;
      [[fallthrough]];                                           // wide rows: AUTO is the split algorithm
    case OMNI_EXPERT_ALGO_SPLIT: {
      int lpr = 0;
      return (split_col_blocks(H, es, &lpr) != 0 && k <= 2 * kWave) ? OMNI_OK : OMNI_ERR_UNSUPPORTED;
    }
    case OMNI_EXPERT_ALGO_GATHER: case OMNI_EXPERT_ALGO_SEGMENT: return (int64_t)H * es <= 8192 ? OMNI_OK : OMNI_ERR_UNSUPPORTED;
    case OMNI_EXPERT_ALGO_DENSE: return (k == 0 || T == 0 || dense_covers(T, H, N, k, dtype)) ? OMNI_OK : OMNI_ERR_UNSUPPORTED;
    default: return OMNI_ERR_UNSUPPORTED;
  }
}

}  // namespace omni

extern "C" OMNI_API size_t omni_expert_workspace_bytes(int64_t num_tokens, int32_t hidden_size, int64_t num_experts,
                                                       int32_t num_experts_per_token, int32_t dtype, int32_t algo) {
  if (num_tokens < 0 || num_experts <= 0 || num_experts_per_token < 0) return 0;
  algo = omni::resolve_algo(algo, num_tokens, hidden_size, num_experts, num_experts_per_token, dtype);
  if (algo == OMNI_EXPERT_ALGO_SPLIT) {
    int lpr = 0;
    const int col_blocks = omni::split_col_blocks(hidden_size, dtype == OMNI_F32 ? 4 : 2, &lpr);
    return omni::align256((size_t)omni::kSlices * (size_t)(col_blocks ? col_blocks : 1) * (size_t)num_tokens * (size_t)num_experts_per_token * 4);
  }
  if (algo == OMNI_EXPERT_ALGO_DENSE)
    return omni::dense_covers(num_tokens, hidden_size, num_experts, num_experts_per_token, dtype) ? omni::dense_workspace_bytes(num_tokens, hidden_size, num_experts) : 0;
  if (algo != OMNI_EXPERT_ALGO_SEGMENT) return 0;   // the gather algorithm keeps everything in registers
  const size_t P = (size_t)num_tokens * (size_t)num_experts_per_token;
  return omni::align256((size_t)(num_experts + 1) * 4) + 2 * omni::align256(P * 4) +
         omni_schedule_workspace_bytes(num_tokens, num_experts_per_token, num_experts);
}

extern "C" OMNI_API int32_t omni_expert_fwd(const void* x, const void* up_weight, const void* down_weight,
                               const void* routing_weights, const int32_t* indices, void* y,
                               int64_t num_tokens, int32_t hidden_size, int64_t num_experts,
                               int32_t num_experts_per_token, int32_t dtype, int32_t algo,
                               void* workspace, void* stream) {
  using namespace omni;
  if (num_tokens < 0 || hidden_size <= 0 || num_experts <= 0 || num_experts_per_token < 0) return OMNI_ERR_SHAPE;
  if (num_tokens > INT32_MAX / 2 || num_experts > UINT32_MAX) return OMNI_ERR_SHAPE;
  if (num_tokens > 0 && (!x || !up_weight || !down_weight || !y)) return OMNI_ERR_NULL;
  if (num_tokens > 0 && num_experts_per_token > 0 && (!routing_weights || !indices)) return OMNI_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  algo = resolve_algo(algo, num_tokens, hidden_size, num_experts, num_experts_per_token, dtype);
  if (algo == OMNI_EXPERT_ALGO_SEGMENT) {
    switch (dtype) {
      case OMNI_BF16: return expert_segment_dispatch<kBF16>(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token, num_experts, workspace, s);
      case OMNI_F16: return expert_segment_dispatch<kF16>(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token, num_experts, workspace, s);
      case OMNI_F32: return expert_segment_dispatch<kF32>(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token, num_experts, workspace, s);
      default: return OMNI_ERR_DTYPE;
    }
  }
  if (algo == OMNI_EXPERT_ALGO_SPLIT) {
    switch (dtype) {
      case OMNI_BF16: return expert_split_dispatch<kBF16>(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token, num_experts, workspace, s);
      case OMNI_F16: return expert_split_dispatch<kF16>(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token, num_experts, workspace, s);
      case OMNI_F32: return expert_split_dispatch<kF32>(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token, num_experts, workspace, s);
      default: return OMNI_ERR_DTYPE;
    }
  }
  if (algo == OMNI_EXPERT_ALGO_DENSE) {
    if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
    if (num_experts_per_token == 0)   // writes zeros
      return omni_expert_fwd(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts, 0, dtype, OMNI_EXPERT_ALGO_GATHER, nullptr, stream);
    return expert_dense_dispatch(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token,
                                 num_experts, dtype, workspace, s);
  }
  if (algo != OMNI_EXPERT_ALGO_GATHER) return OMNI_ERR_UNSUPPORTED;
  switch (dtype) {
    case OMNI_BF16: return expert_gather_dispatch<kBF16>(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token, num_experts, s);
    case OMNI_F16: return expert_gather_dispatch<kF16>(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token, num_experts, s);
    case OMNI_F32: return expert_gather_dispatch<kF32>(x, up_weight, down_weight, routing_weights, indices, y, num_tokens, hidden_size, num_experts_per_token, num_experts, s);
    default: return OMNI_ERR_DTYPE;
  }
}
