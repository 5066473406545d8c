// Backward kernels of the three OmniMoE operators for gfx950, so that a layer built on them
// trains.  Each replaces the matching Triton backward of the reference:
//   * router   (omni_moe/ops/triton/omni_router.py:98-164, 235-274): the gradient of the k
//     selected scores scatters back to the two half-logit rows, d_lx[ix] += ds, d_ly[iy] += ds;
//   * experts  (omni_expert.py:375-618, 1067-1277): for a pair (t, e) with s = <x_t, U_e>,
//     a = <dy_t, V_e>:   dg = a silu(s),   ds = a g silu'(s),   dx_t += ds U_e,
//     dU_e += ds x_t,   dV_e += silu(s) g dy_t;
//   * SwiGLU   (omni_mlp.py:102-177 forward, 180-249 backward) as element-wise kernels for
//     the training path, which keeps gate and up (the inference path forms the product in the
//     GEMM epilogue and never stores them).
// All sums are fp32 in a fixed order, rounded once on the way out: no atomics anywhere (the
// reference accumulates dx, dU and dV with atomics in the storage dtype), so gradients are
// run-to-run identical.
//
// Expert backward in two passes.  Token pass: one wave owns one token, keeps x_t, dy_t and the
// fp32 dx accumulator in registers, fetches each selected up and down row once, recomputes s
// (nothing is saved by the forward), writes dg and, to an fp32 workspace, ds and the forward
// coefficient silu(s) g of every pair.  Weight pass: the pairs are grouped by expert with the
// stable schedule of the forward path; one wave owns one expert, walks its segment and gathers
// the x and dy rows of the segment's tokens, so every dU/dV row is written exactly once
// (zeros for experts nobody selected).
#include "common.h"
#include "omni_moe_hip.h"
#include "rows.h"

namespace omni {

constexpr int kBwdWavesPerBlock = 4;

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + __expf(-x)); }

// ---- router ------------------------------------------------------------------------------------
// One wave per token; lane l accumulates columns l, l+64, ... of both halves (r <= 64 * kCols).
template <int DT, int kCols>
__global__ __launch_bounds__(kBwdWavesPerBlock* kWave) void router_bwd_kernel(
    const void* __restrict__ dscores, const int32_t* __restrict__ ids, void* __restrict__ dlx, void* __restrict__ dly,
    int num_tokens, int r, int top_k) {
  const int lane = lane_id();
  const int t = __builtin_amdgcn_readfirstlane(blockIdx.x * kBwdWavesPerBlock + (threadIdx.x >> 6));
  if (t >= num_tokens) return;
  float ax[kCols], ay[kCols];
#pragma unroll
  for (int c = 0; c < kCols; ++c) ax[c] = ay[c] = 0.f;
  const int64_t base = int64_t(t) * top_k;
  for (int j0 = 0; j0 < top_k; j0 += kWave) {       // k <= 128: at most two rounds
    const int j = j0 + lane;
    const int my_id = j < top_k ? ids[base + j] : -1;
    const float my_ds = j < top_k ? Elem<DT>::load(dscores, base + j) : 0.f;
    // lane j splits slot j's id once; an id outside the product gets coordinates no lane owns
    const bool ok = (uint32_t)my_id < (uint32_t)r * (uint32_t)r;
    const int my_ix = ok ? my_id / r : -1, my_iy = ok ? my_id - my_ix * r : -1;
    const int n = min(kWave, top_k - j0);
    for (int i = 0; i < n; ++i) {                   // slot order: the sum per column is deterministic
      const int ix = __shfl(my_ix, i, kWave), iy = __shfl(my_iy, i, kWave);
      const float ds = __shfl(my_ds, i, kWave);
#pragma unroll
      for (int c = 0; c < kCols; ++c) {
        ax[c] += (ix == c * kWave + lane) ? ds : 0.f;
        ay[c] += (iy == c * kWave + lane) ? ds : 0.f;
      }
    }
  }
#pragma unroll
  for (int c = 0; c < kCols; ++c) {
    const int col = c * kWave + lane;
    if (col < r) {
      Elem<DT>::store(dlx, int64_t(t) * r + col, ax[c]);
      Elem<DT>::store(dly, int64_t(t) * r + col, ay[c]);
    }
  }
}

// ---- router stage: exp, Cartesian select, log-softmax and BatchNorm in reverse -------------------
// The layer's router forward (omni_moe.py:70-86) is  z = x W^T -> n = BN(z) -> l = log_softmax(n)
// -> scores = lx[ix] + ly[iy] -> gates = exp(scores).  Given d(gates), this pass returns d(z); the
// two GEMMs around it (dW = dz^T x, dx = dz W) are the caller's.  One wave owns a token and walks
// both halves with lane = column (R columns per lane and half):
//   d(score_j) = d(gate_j) gate_j;  d(l) = scatter of d(score) by (ix, iy), in slot order;
//   d(n) = d(l) - exp(l) sum(d(l));                      (log-softmax)
//   eval:  d(z) = rstd d(n);   train:  d(z) = rstd (d(n) - mean_T d(n) - nhat mean_T(d(n) nhat)).
// Training needs the two column means over all tokens: the first kernel leaves d(n) in the dz
// buffer and per-block column sums, a one-wave-per-column kernel adds those, a third kernel
// finishes d(z).  Values are rounded to the storage dtype where the reference's torch ops round
// (d(score), d(l), d(n), d(z)); n and l are recomputed from z and the saved statistics.
constexpr int kNormTokensPerWave = 8;

template <int DT, int R>
__global__ __launch_bounds__(kBwdWavesPerBlock* kWave) void router_norm_bwd_kernel(
    const void* __restrict__ dgates, const void* __restrict__ gates, const int32_t* __restrict__ ids,
    const void* __restrict__ z, const float* __restrict__ stats, void* __restrict__ dz, float* __restrict__ partials,
    int num_tokens, int r, int top_k, int training) {
  __shared__ float red[kBwdWavesPerBlock][4][R * kWave];       // per wave: S1x, S2x, S1y, S2y by column
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  const int first = (blockIdx.x * kBwdWavesPerBlock + wave) * kNormTokensPerWave;
  float s1[2][R], s2[2][R];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int a = 0; a < R; ++a) s1[h][a] = s2[h][a] = 0.f;
  float mean[2][R], rstd[2][R];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int a = 0; a < R; ++a) {
      const int key = a * kWave + lane;
      mean[h][a] = key < r ? stats[(2 * h) * r + key] : 0.f;
      rstd[h][a] = key < r ? stats[(2 * h + 1) * r + key] : 0.f;
    }
  for (int t = first; t < min(first + kNormTokensPerWave, num_tokens); ++t) {
    // d(l): scatter of the slot gradients, fp32 sums in slot order, one rounding
    float dl[2][R];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int a = 0; a < R; ++a) dl[h][a] = 0.f;
    const int64_t base = int64_t(t) * top_k;
    for (int j0 = 0; j0 < top_k; j0 += kWave) {
      const int j = j0 + lane;
      const int my_id = j < top_k ? ids[base + j] : -1;
      const float my_ds = j < top_k ? Elem<DT>::round(Elem<DT>::load(dgates, base + j) * Elem<DT>::load(gates, base + j)) : 0.f;
      const bool ok = (uint32_t)my_id < (uint32_t)r * (uint32_t)r;
      const int my_ix = ok ? my_id / r : -1, my_iy = ok ? my_id - my_ix * r : -1;
      const int n = min(kWave, top_k - j0);
      for (int i = 0; i < n; ++i) {
        const int ix = __shfl(my_ix, i, kWave), iy = __shfl(my_iy, i, kWave);
        const float ds = __shfl(my_ds, i, kWave);
#pragma unroll
        for (int a = 0; a < R; ++a) {
          dl[0][a] += (ix == a * kWave + lane) ? ds : 0.f;
          dl[1][a] += (iy == a * kWave + lane) ? ds : 0.f;
        }
      }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      // recompute nhat (fp32), n = round(nhat), l = round(log_softmax(n))
      float nhat[R], l[R];
      float m = -INFINITY;
#pragma unroll
      for (int a = 0; a < R; ++a) {
        const int key = a * kWave + lane;
        const float zv = key < r ? Elem<DT>::load(z, int64_t(t) * 2 * r + h * r + key) : 0.f;
        nhat[a] = (zv - mean[h][a]) * rstd[h][a];
        l[a] = key < r ? Elem<DT>::round(nhat[a]) : -INFINITY;
        m = fmaxf(m, l[a]);
      }
      m = wave_max(m);
      float e = 0.f;
#pragma unroll
      for (int a = 0; a < R; ++a) e += (a * kWave + lane < r) ? expf(l[a] - m) : 0.f;
      const float lse = logf(wave_sum(e));
      float sum_dl = 0.f;
#pragma unroll
      for (int a = 0; a < R; ++a) {
        dl[h][a] = Elem<DT>::round(dl[h][a]);
        sum_dl += dl[h][a];
      }
      sum_dl = wave_sum(sum_dl);
#pragma unroll
      for (int a = 0; a < R; ++a) {
        const int key = a * kWave + lane;
        if (key >= r) continue;
        const float p = expf(Elem<DT>::round(l[a] - m - lse));
        const float dn = Elem<DT>::round(dl[h][a] - p * sum_dl);
        s1[h][a] += dn;
        s2[h][a] += dn * nhat[a];
        Elem<DT>::store(dz, int64_t(t) * 2 * r + h * r + key, training ? dn : dn * rstd[h][a]);
      }
    }
  }
  if (!training) return;
  // column sums of the block: waves in order through LDS, then one row of partials per block
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int a = 0; a < R; ++a) {
      red[wave][2 * h][a * kWave + lane] = s1[h][a];
      red[wave][2 * h + 1][a * kWave + lane] = s2[h][a];
    }
  __syncthreads();
  for (int i = threadIdx.x; i < 4 * R * kWave; i += kBwdWavesPerBlock * kWave) {
    const int q = i / (R * kWave), col = i % (R * kWave);
    if (col >= r) continue;
    float acc = 0.f;
#pragma unroll
    for (int w = 0; w < kBwdWavesPerBlock; ++w) acc += red[w][q][col];
    partials[(int64_t(blockIdx.x) * 4 + q) * r + col] = acc;     // [block][S1x, S2x, S1y, S2y][r]
  }
}

// means[q][col] = sum over blocks of partials / T; one wave per (q, col)
__global__ __launch_bounds__(kBwdWavesPerBlock* kWave) void router_norm_bwd_sums_kernel(
    const float* __restrict__ partials, float* __restrict__ means, int blocks, int r, int num_tokens) {
  const int lane = lane_id();
  const int idx = blockIdx.x * kBwdWavesPerBlock + (threadIdx.x >> 6);      // q * r + col
  if (idx >= 4 * r) return;
  double acc = 0.;
  for (int b = lane; b < blocks; b += kWave) acc += (double)partials[int64_t(b) * 4 * r + idx];
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, kWave);
  if (lane == 0) means[idx] = (float)(acc / (double)num_tokens);
}

// dz = rstd (dn - mean(dn) - nhat mean(dn nhat)), element-wise over [T, 2r]; dn is read from dz
template <int DT>
__global__ __launch_bounds__(256) void router_norm_bwd_finish_kernel(const void* __restrict__ z, const float* __restrict__ stats,
                                                                    const float* __restrict__ means, void* __restrict__ dz,
                                                                    int64_t num_values, int r) {
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < num_values; i += gridDim.x * 256ll) {
    const int c = (int)(i % (2 * r)), h = c >= r, key = c - h * r;
    const float mu = stats[(2 * h) * r + key], rs = stats[(2 * h + 1) * r + key];
    const float nhat = (Elem<DT>::load(z, i) - mu) * rs;
    const float dn = Elem<DT>::load(dz, i);
    Elem<DT>::store(dz, i, rs * (dn - means[(2 * h) * r + key] - nhat * means[(2 * h + 1) * r + key]));
  }
}

// ---- experts, token pass -----------------------------------------------------------------------
template <int DT, int NCH, int G>
__global__ __launch_bounds__(kBwdWavesPerBlock* kWave, 2) void expert_bwd_token_kernel(
    const uint8_t* __restrict__ x, const uint8_t* __restrict__ dy, const uint8_t* __restrict__ up,
    const uint8_t* __restrict__ down, const void* __restrict__ gates, const int32_t* __restrict__ ids,
    uint8_t* __restrict__ dx, void* __restrict__ dgates, float* __restrict__ ds_out, float* __restrict__ coef_out,
    int num_tokens, int hidden, int top_k, uint32_t num_experts) {
  constexpr int E = Row16<DT>::kElems;
  const int lane = lane_id();
  const int t = __builtin_amdgcn_readfirstlane(blockIdx.x * kBwdWavesPerBlock + (threadIdx.x >> 6));
  if (t >= num_tokens) return;
  const int64_t row_bytes = int64_t(hidden) * (16 / E);

  bool live[NCH];
  int64_t off[NCH];
  u32x4_t xr[NCH], dyr[NCH];
  float acc[NCH][E];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    live[c] = (c * kWave + lane) * E < hidden;
    off[c] = int64_t(c * kWave + lane) * 16;
    xr[c] = live[c] ? *(const u32x4_t*)(x + t * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};
    dyr[c] = live[c] ? *(const u32x4_t*)(dy + t * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < E; ++i) acc[c][i] = 0.f;
  }

  const int64_t base = int64_t(t) * top_k;
  for (int j0 = 0; j0 < top_k; j0 += G) {
    int e[G];
    float g[G];
    bool live_slot[G];
#pragma unroll
    for (int i = 0; i < G; ++i) {
      const int j = min(j0 + i, top_k - 1);
      const int id = ids[base + j];
      const float gate = Elem<DT>::load(gates, base + j);
      const bool ok = (j0 + i < top_k) && (uint32_t)id < num_experts;   // as the forward: such a pair contributes nothing
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

    float s[G], a[G];
#pragma unroll
    for (int i = 0; i < G; ++i) {
      float ps = 0.f, pa = 0.f;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        ps = dot16<DT>(xr[c], ur[i][c], ps);
        pa = dot16<DT>(dyr[c], vr[i][c], pa);
      }
      s[i] = ps;
      a[i] = pa;
    }
#pragma unroll
    for (int i = 0; i < G; ++i) {
      s[i] = wave_sum(s[i]);
      a[i] = wave_sum(a[i]);
    }
#pragma unroll
    for (int i = 0; i < G; ++i) {
      const float sig = sigmoid_f32(s[i]);
      const float silu = s[i] * sig;
      const float dsilu = sig + silu * (1.0f - sig);
      const float dg = live_slot[i] ? a[i] * silu : 0.f;
      const float ds = live_slot[i] ? a[i] * g[i] * dsilu : 0.f;
      const float coef = live_slot[i] ? silu * g[i] : 0.f;
      if (lane == 0 && j0 + i < top_k) {
        Elem<DT>::store(dgates, base + j0 + i, dg);
        ds_out[base + j0 + i] = ds;
        coef_out[base + j0 + i] = coef;
      }
      if (live_slot[i]) {                       // not even 0 * row: the stand-in row may hold Inf or NaN
#pragma unroll
        for (int c = 0; c < NCH; ++c) axpy16<DT>(ds, ur[i][c], acc[c]);
      }
    }
  }
#pragma unroll
  for (int c = 0; c < NCH; ++c)
    if (live[c]) *(u32x4_t*)(dx + t * row_bytes + off[c]) = pack16<DT>(acc[c]);
}

// ---- experts, weight pass ----------------------------------------------------------------------
// The sorted pair list is cut into chunks of `chunk` consecutive pairs, one wave each, whatever the
// segment lengths: a popular expert's segment is spread over many waves and many rare experts
// share one.  Inside its chunk a wave sums run after run (a run = the chunk's pairs of one
// expert).  A run that is the expert's whole segment is rounded and stored straight away.  A run
// of a segment that crosses the chunk's border is left as an fp32 partial row pair in
// `partials[chunk][slot]`, slot 0 if the run starts the chunk, slot 1 otherwise (a chunk has at
// most one of each); the fix-up kernel then adds an expert's partials in chunk order, so the
// summation order is fixed and nothing is added atomically.
template <int DT, int NCH, int G>
__global__ __launch_bounds__(kBwdWavesPerBlock* kWave, 2) void expert_bwd_weight_kernel(
    const uint8_t* __restrict__ x, const uint8_t* __restrict__ dy, const float* __restrict__ ds, const float* __restrict__ coef,
    const int32_t* __restrict__ ids, const int32_t* __restrict__ offsets, const int32_t* __restrict__ sorted_pair_ids,
    const int32_t* __restrict__ sorted_token_ids, uint8_t* __restrict__ dup, uint8_t* __restrict__ ddown,
    float* __restrict__ partials, int64_t num_experts, int hidden, int chunk, int num_chunks) {
  constexpr int E = Row16<DT>::kElems;
  const int lane = lane_id();
  const int ci = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * kBwdWavesPerBlock + (threadIdx.x >> 6)));
  if (ci >= num_chunks) return;
  const int valid = offsets[num_experts];             // pairs with an id inside the table
  const int first = ci * chunk, last = min(first + chunk, valid);
  if (first >= last) return;
  const int64_t row_bytes = int64_t(hidden) * (16 / E);

  bool live[NCH];
  int64_t off[NCH];
  float au[NCH][E], av[NCH][E];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    live[c] = (c * kWave + lane) * E < hidden;
    off[c] = int64_t(c * kWave + lane) * 16;
#pragma unroll
    for (int i = 0; i < E; ++i) au[c][i] = av[c][i] = 0.f;
  }
  // ends the run [run_first, run_last) of expert e and clears the accumulators
  auto flush = [&](int e, int run_first, int run_last) {
    const bool whole = offsets[e] == run_first && offsets[e + 1] == run_last;
    if (whole) {
#pragma unroll
      for (int c = 0; c < NCH; ++c)
        if (live[c]) {
          *(u32x4_t*)(dup + e * row_bytes + off[c]) = pack16<DT>(au[c]);
          *(u32x4_t*)(ddown + e * row_bytes + off[c]) = pack16<DT>(av[c]);
        }
    } else {
      float* out = partials + (int64_t(ci) * 2 + (run_first == first ? 0 : 1)) * 2 * hidden;
#pragma unroll
      for (int c = 0; c < NCH; ++c)
        if (live[c]) {
          const int col = (c * kWave + lane) * E;
#pragma unroll
          for (int q = 0; q < E; q += 4) {
            *(f32x4_t*)(out + col + q) = f32x4_t{au[c][q], au[c][q + 1], au[c][q + 2], au[c][q + 3]};
            *(f32x4_t*)(out + hidden + col + q) = f32x4_t{av[c][q], av[c][q + 1], av[c][q + 2], av[c][q + 3]};
          }
        }
    }
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
      for (int i = 0; i < E; ++i) au[c][i] = av[c][i] = 0.f;
  };

  int run_e = __builtin_amdgcn_readfirstlane(ids[sorted_pair_ids[first]]), run_first = first;
  for (int p0 = first; p0 < last; p0 += G) {          // list order = (expert, pair) order: a fixed summation order
    int64_t tok[G];
    int ee[G];
    float cs[G], cc[G];
#pragma unroll
    for (int i = 0; i < G; ++i) {
      const int p = min(p0 + i, last - 1);
      const int pid = sorted_pair_ids[p];
      tok[i] = sorted_token_ids[p];
      ee[i] = __builtin_amdgcn_readfirstlane(ids[pid]);
      cs[i] = ds[pid];
      cc[i] = coef[pid];
    }
    u32x4_t xr[G][NCH], dyr[G][NCH];
#pragma unroll
    for (int i = 0; i < G; ++i)
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        xr[i][c] = live[c] ? *(const u32x4_t*)(x + tok[i] * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};
        dyr[i][c] = live[c] ? *(const u32x4_t*)(dy + tok[i] * row_bytes + off[c]) : u32x4_t{0, 0, 0, 0};
      }
#pragma unroll
    for (int i = 0; i < G; ++i) {
      if (p0 + i >= last) break;
      if (ee[i] != run_e) {
        flush(run_e, run_first, p0 + i);
        run_e = ee[i];
        run_first = p0 + i;
      }
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        axpy16<DT>(cs[i], xr[i][c], au[c]);
        axpy16<DT>(cc[i], dyr[i][c], av[c]);
      }
    }
  }
  flush(run_e, run_first, last);
}

// One wave per expert: zero rows for an expert nobody selected; for a segment that crosses a chunk
// border the sum of its partial rows, first chunk to last.  A segment inside one chunk was
// stored by the pass above.
template <int DT, int NCH>
__global__ __launch_bounds__(kBwdWavesPerBlock* kWave) void expert_bwd_weight_fixup_kernel(
    const int32_t* __restrict__ offsets, const float* __restrict__ partials, uint8_t* __restrict__ dup,
    uint8_t* __restrict__ ddown, int64_t num_experts, int hidden, int chunk) {
  constexpr int E = Row16<DT>::kElems;
  const int lane = lane_id();
  const int64_t e = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * kBwdWavesPerBlock + (threadIdx.x >> 6)));
  if (e >= num_experts) return;
  const int begin = offsets[e], end = offsets[e + 1];
  const int c0 = begin / chunk, c1 = end > begin ? (end - 1) / chunk : c0;
  if (end > begin && c0 == c1) return;
  const int64_t row_bytes = int64_t(hidden) * (16 / E);
  float au[NCH][E], av[NCH][E];
#pragma unroll
  for (int c = 0; c < NCH; ++c)
#pragma unroll
    for (int i = 0; i < E; ++i) au[c][i] = av[c][i] = 0.f;
  if (end > begin) {
    for (int ci = c0; ci <= c1; ++ci) {
      const int slot = (ci == c0 && begin != c0 * chunk) ? 1 : 0;
      const float* in = partials + (int64_t(ci) * 2 + slot) * 2 * hidden;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int col = (c * kWave + lane) * E;
        if (col < hidden) {
#pragma unroll
          for (int q = 0; q < E; q += 4) {
            const f32x4_t u = *(const f32x4_t*)(in + col + q), v = *(const f32x4_t*)(in + hidden + col + q);
#pragma unroll
            for (int z = 0; z < 4; ++z) {
              au[c][q + z] += u[z];
              av[c][q + z] += v[z];
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int c = 0; c < NCH; ++c)
    if ((c * kWave + lane) * E < hidden) {
      *(u32x4_t*)(dup + e * row_bytes + int64_t(c * kWave + lane) * 16) = pack16<DT>(au[c]);
      *(u32x4_t*)(ddown + e * row_bytes + int64_t(c * kWave + lane) * 16) = pack16<DT>(av[c]);
    }
}

// ---- SwiGLU, element-wise ----------------------------------------------------------------------
// 16 bytes per lane.  Forward: out = silu(gate) * up in fp32, one rounding (omni_mlp.py:53-61).
// Backward: with a = gate in fp32, sig = sigmoid(a):  d_up = dout * a sig,
// d_gate = dout * (a sig (1 - sig) + sig) * up  (omni_mlp.py:232-236).
template <int DT, bool BWD>
__global__ __launch_bounds__(256) void swiglu_kernel(const uint8_t* __restrict__ dout, const uint8_t* __restrict__ gate,
                                                    const uint8_t* __restrict__ up, uint8_t* __restrict__ out0,
                                                    uint8_t* __restrict__ out1, int64_t num_chunks) {
  constexpr int E = Row16<DT>::kElems;
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < num_chunks; i += gridDim.x * 256ll) {
    const u32x4_t gw = *(const u32x4_t*)(gate + i * 16), uw = *(const u32x4_t*)(up + i * 16);
    float gv[E], uv[E], r0[E], r1[E];
    unpack16<DT>(gw, gv);
    unpack16<DT>(uw, uv);
    if constexpr (BWD) {
      float dv[E];
      unpack16<DT>(*(const u32x4_t*)(dout + i * 16), dv);
#pragma unroll
      for (int q = 0; q < E; ++q) {
        const float sig = sigmoid_f32(gv[q]), silu = gv[q] * sig;
        r0[q] = dv[q] * (silu * (1.0f - sig) + sig) * uv[q];
        r1[q] = dv[q] * silu;
      }
      *(u32x4_t*)(out0 + i * 16) = pack16<DT>(r0);
      *(u32x4_t*)(out1 + i * 16) = pack16<DT>(r1);
    } else {
#pragma unroll
      for (int q = 0; q < E; ++q) r0[q] = gv[q] * sigmoid_f32(gv[q]) * uv[q];
      *(u32x4_t*)(out0 + i * 16) = pack16<DT>(r0);
    }
  }
}

// ---- host side ---------------------------------------------------------------------------------
static inline size_t up256(size_t v) { return (v + 255) / 256 * 256; }
static int to_code(hipError_t e) { return e == hipSuccess ? OMNI_OK : OMNI_ERR_HIP_BASE + (int)e; }

// pairs per weight-pass chunk: about 2048 chunks (8 waves per CU), at least 16 pairs each
static inline int weight_chunk(size_t pairs) {
  const size_t c = (pairs + 2047) / 2048;
  return (int)(c < 16 ? 16 : c);
}

template <int DT, int NCH, int G>
static hipError_t launch_expert_bwd(const void* dy, const void* x, const void* up, const void* down, const void* gates,
                                    const int32_t* ids, void* dx, void* dup, void* ddown, void* dgates, float* ds, float* coef,
                                    const int32_t* offsets, const int32_t* pair_ids, const int32_t* token_ids, float* partials,
                                    int64_t T, int H, int64_t N, int k, hipStream_t s) {
  dim3 block(kBwdWavesPerBlock * kWave);
  if (T > 0) {
    dim3 grid((unsigned)((T + kBwdWavesPerBlock - 1) / kBwdWavesPerBlock));
    hipLaunchKernelGGL((expert_bwd_token_kernel<DT, NCH, G>), grid, block, 0, s, (const uint8_t*)x, (const uint8_t*)dy,
                       (const uint8_t*)up, (const uint8_t*)down, gates, ids, (uint8_t*)dx, dgates, ds, coef, (int)T, H, k,
                       (uint32_t)N);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
  }
  const size_t P = (size_t)T * (size_t)k;
  const int chunk = weight_chunk(P);
  const int num_chunks = (int)((P + chunk - 1) / chunk);
  if (num_chunks > 0) {
    dim3 grid((unsigned)((num_chunks + kBwdWavesPerBlock - 1) / kBwdWavesPerBlock));
    hipLaunchKernelGGL((expert_bwd_weight_kernel<DT, NCH, G>), grid, block, 0, s, (const uint8_t*)x, (const uint8_t*)dy, ds, coef,
                       ids, offsets, pair_ids, token_ids, (uint8_t*)dup, (uint8_t*)ddown, partials, N, H, chunk, num_chunks);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
  }
  dim3 grid((unsigned)((N + kBwdWavesPerBlock - 1) / kBwdWavesPerBlock));
  hipLaunchKernelGGL((expert_bwd_weight_fixup_kernel<DT, NCH>), grid, block, 0, s, offsets, partials, (uint8_t*)dup,
                     (uint8_t*)ddown, N, H, chunk);
  return hipGetLastError();
}

}  // namespace omni

extern "C" OMNI_API int32_t omni_router_bwd(const void* dscores, const int32_t* indices, void* dlogits_x, void* dlogits_y,
                                            int64_t num_tokens, int32_t num_expert_sqrt, int32_t num_experts_per_token,
                                            int32_t dtype, void* stream) {
  using namespace omni;
  if (num_tokens < 0 || num_tokens > INT32_MAX || num_expert_sqrt <= 0 || num_experts_per_token < 0) return OMNI_ERR_SHAPE;
  if (num_expert_sqrt > 1024) return OMNI_ERR_UNSUPPORTED;
  if (num_experts_per_token > 128) return OMNI_ERR_TOPK;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  if (num_tokens == 0) return OMNI_OK;
  if (!dlogits_x || !dlogits_y || (num_experts_per_token > 0 && (!dscores || !indices))) return OMNI_ERR_NULL;
  dim3 grid((unsigned)((num_tokens + kBwdWavesPerBlock - 1) / kBwdWavesPerBlock)), block(kBwdWavesPerBlock * kWave);
  hipStream_t s = (hipStream_t)stream;
  const int T = (int)num_tokens, r = num_expert_sqrt, k = num_experts_per_token;
#define OMNI_ROUTER_BWD_CASE(DT)                                                                                             \
  do {                                                                                                                       \
    if (r <= 64) hipLaunchKernelGGL((router_bwd_kernel<DT, 1>), grid, block, 0, s, dscores, indices, dlogits_x, dlogits_y, T, r, k);        \
    else if (r <= 256) hipLaunchKernelGGL((router_bwd_kernel<DT, 4>), grid, block, 0, s, dscores, indices, dlogits_x, dlogits_y, T, r, k);  \
    else hipLaunchKernelGGL((router_bwd_kernel<DT, 16>), grid, block, 0, s, dscores, indices, dlogits_x, dlogits_y, T, r, k);               \
  } while (0)
  if (dtype == OMNI_BF16) OMNI_ROUTER_BWD_CASE(kBF16);
  else if (dtype == OMNI_F16) OMNI_ROUTER_BWD_CASE(kF16);
  else OMNI_ROUTER_BWD_CASE(kF32);
#undef OMNI_ROUTER_BWD_CASE
  return to_code(hipGetLastError());
}

// workspace of omni_router_norm_bwd: per-block column sums [blocks][4][r] f32 | means [4][r] f32
static inline int norm_bwd_blocks(int64_t num_tokens) {
  const int64_t per_block = (int64_t)omni::kBwdWavesPerBlock * omni::kNormTokensPerWave;
  return (int)((num_tokens + per_block - 1) / per_block);
}

extern "C" OMNI_API size_t omni_router_norm_bwd_workspace_bytes(int64_t num_tokens, int32_t num_expert_sqrt) {
  using namespace omni;
  if (num_tokens < 0 || num_expert_sqrt <= 0) return 0;
  return up256((size_t)norm_bwd_blocks(num_tokens) * 4 * num_expert_sqrt * 4) + up256((size_t)4 * num_expert_sqrt * 4);
}

extern "C" OMNI_API int32_t omni_router_norm_bwd(const void* dgates, const void* gates, const int32_t* indices, const void* z,
                                                 const float* stats, void* dz, int64_t num_tokens, int32_t num_expert_sqrt,
                                                 int32_t num_experts_per_token, int32_t dtype, int32_t training, void* workspace,
                                                 void* stream) {
  using namespace omni;
  const int r = num_expert_sqrt, k = num_experts_per_token;
  if (num_tokens < 0 || num_tokens > INT32_MAX / 4096 || r <= 0 || k < 0) return OMNI_ERR_SHAPE;
  if (r > 1024) return OMNI_ERR_UNSUPPORTED;
  if (k > 128) return OMNI_ERR_TOPK;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  if (num_tokens == 0) return OMNI_OK;
  if (!z || !stats || !dz || (k > 0 && (!dgates || !gates || !indices))) return OMNI_ERR_NULL;
  if (training && !workspace) return OMNI_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  const int T = (int)num_tokens, blocks = norm_bwd_blocks(num_tokens);
  float* partials = (float*)workspace;
  float* means = training ? (float*)((char*)workspace + up256((size_t)blocks * 4 * r * 4)) : nullptr;
  dim3 block(kBwdWavesPerBlock * kWave);
#define OMNI_NORM_CASE(DT)                                                                                                    \
  do {                                                                                                                        \
    if (r <= 64) hipLaunchKernelGGL((router_norm_bwd_kernel<DT, 1>), dim3(blocks), block, 0, s, dgates, gates, indices, z,     \
                                    stats, dz, partials, T, r, k, training);                                                   \
    else if (r <= 256) hipLaunchKernelGGL((router_norm_bwd_kernel<DT, 4>), dim3(blocks), block, 0, s, dgates, gates, indices,  \
                                          z, stats, dz, partials, T, r, k, training);                                          \
    else hipLaunchKernelGGL((router_norm_bwd_kernel<DT, 16>), dim3(blocks), block, 0, s, dgates, gates, indices, z, stats, dz, \
                            partials, T, r, k, training);                                                                      \
    if (training) {                                                                                                           \
      hipLaunchKernelGGL(router_norm_bwd_sums_kernel, dim3((4 * r + kBwdWavesPerBlock - 1) / kBwdWavesPerBlock), block, 0, s,  \
                         partials, means, blocks, r, T);                                                                       \
      const int64_t values = (int64_t)T * 2 * r;                                                                              \
      const int64_t want = (values + 255) / 256;                                                                              \
      hipLaunchKernelGGL(router_norm_bwd_finish_kernel<DT>, dim3((unsigned)(want < 4096 ? want : 4096)), dim3(256), 0, s, z,   \
                         stats, means, dz, values, r);                                                                         \
    }                                                                                                                         \
  } while (0)
  if (dtype == OMNI_BF16) OMNI_NORM_CASE(kBF16);
  else if (dtype == OMNI_F16) OMNI_NORM_CASE(kF16);
  else OMNI_NORM_CASE(kF32);
#undef OMNI_NORM_CASE
  return to_code(hipGetLastError());
}

// workspace: ds [P] f32 | coef [P] f32 | sorted pair ids [P] i32 | sorted token ids [P] i32 | offsets [N+1] i32 |
//            partial rows [chunks][2][2][H] f32 | schedule workspace
extern "C" OMNI_API size_t omni_expert_bwd_workspace_bytes(int64_t num_tokens, int32_t hidden_size, int64_t num_experts,
                                                           int32_t num_experts_per_token, int32_t dtype) {
  using namespace omni;
  (void)dtype;
  if (num_tokens < 0 || num_experts <= 0 || num_experts_per_token < 0 || hidden_size <= 0) return 0;
  const size_t P = (size_t)num_tokens * (size_t)num_experts_per_token;
  const size_t chunks = (P + weight_chunk(P) - 1) / weight_chunk(P);
  return 4 * up256(P * 4) + up256(((size_t)num_experts + 1) * 4) + up256(chunks * 4 * (size_t)hidden_size * 4) +
         omni_schedule_workspace_bytes(num_tokens, num_experts_per_token, num_experts);
}

extern "C" OMNI_API int32_t omni_expert_bwd(const void* dy, const void* x, const void* up_weight, const void* down_weight,
                                            const void* routing_weights, const int32_t* indices, void* dx, void* dup_weight,
                                            void* ddown_weight, void* drouting_weights, int64_t num_tokens, int32_t hidden_size,
                                            int64_t num_experts, int32_t num_experts_per_token, int32_t dtype, void* workspace,
                                            void* stream) {
  using namespace omni;
  if (num_tokens < 0 || hidden_size <= 0 || num_experts <= 0 || num_experts_per_token < 0) return OMNI_ERR_SHAPE;
  if (num_tokens > INT32_MAX / 2 || num_experts > INT32_MAX / 2 ||
      num_tokens * (int64_t)num_experts_per_token > INT32_MAX / 2)
    return OMNI_ERR_SHAPE;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  if (!dup_weight || !ddown_weight) return OMNI_ERR_NULL;
  if (num_tokens > 0 && (!dy || !x || !dx || !up_weight || !down_weight)) return OMNI_ERR_NULL;
  if (num_tokens > 0 && num_experts_per_token > 0 && (!routing_weights || !indices || !drouting_weights)) return OMNI_ERR_NULL;
  if (!workspace) return OMNI_ERR_WORKSPACE;
  const int E = dtype == OMNI_F32 ? 4 : 8;
  if (hidden_size % E != 0) return OMNI_ERR_SHAPE;
  const int nch = (hidden_size + kWave * E - 1) / (kWave * E);
  if (nch > 8) return OMNI_ERR_UNSUPPORTED;
  const size_t P = (size_t)num_tokens * (size_t)num_experts_per_token;
  char* w = (char*)workspace;
  float* ds = (float*)w;               w += up256(P * 4);
  float* coef = (float*)w;             w += up256(P * 4);
  int32_t* pair_ids = (int32_t*)w;     w += up256(P * 4);
  int32_t* token_ids = (int32_t*)w;    w += up256(P * 4);
  int32_t* offsets = (int32_t*)w;      w += up256(((size_t)num_experts + 1) * 4);
  float* partials = (float*)w;
  {
    const size_t chunks = (P + weight_chunk(P) - 1) / weight_chunk(P);
    w += up256(chunks * 4 * (size_t)hidden_size * 4);
  }
  hipStream_t s = (hipStream_t)stream;
  if (int e = omni_schedule(indices, offsets, pair_ids, token_ids, num_tokens, num_experts_per_token, num_experts, w, stream)) return e;
  const int64_t T = num_tokens, N = num_experts;
  const int H = hidden_size, k = num_experts_per_token;
  hipError_t err;
#define OMNI_BWD_ARGS                                                                                                   \
  dy, x, up_weight, down_weight, routing_weights, indices, dx, dup_weight, ddown_weight, drouting_weights, ds, coef, offsets, \
      pair_ids, token_ids, partials, T, H, N, k, s
#define OMNI_BWD_CASE(DT)                                                      \
  do {                                                                         \
    if (nch <= 1) err = launch_expert_bwd<DT, 1, 8>(OMNI_BWD_ARGS);            \
    else if (nch <= 2) err = launch_expert_bwd<DT, 2, 8>(OMNI_BWD_ARGS);       \
    else if (nch <= 4) err = launch_expert_bwd<DT, 4, 4>(OMNI_BWD_ARGS);       \
    else err = launch_expert_bwd<DT, 8, 2>(OMNI_BWD_ARGS);                     \
  } while (0)
  if (dtype == OMNI_BF16) OMNI_BWD_CASE(kBF16);
  else if (dtype == OMNI_F16) OMNI_BWD_CASE(kF16);
  else OMNI_BWD_CASE(kF32);
#undef OMNI_BWD_ARGS
#undef OMNI_BWD_CASE
  return to_code(err);
}

static int32_t swiglu_launch(bool bwd, const void* dout, const void* gate, const void* up, void* out0, void* out1,
                             int64_t num_elements, int32_t dtype, void* stream) {
  using namespace omni;
  if (num_elements < 0) return OMNI_ERR_SHAPE;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  const int E = dtype == OMNI_F32 ? 4 : 8;
  if (num_elements % E != 0) return OMNI_ERR_SHAPE;
  if (num_elements == 0) return OMNI_OK;
  if (!gate || !up || !out0 || (bwd && (!dout || !out1))) return OMNI_ERR_NULL;
  const int64_t chunks = num_elements / E;
  const int64_t want = (chunks + 255) / 256;
  dim3 grid((unsigned)(want < 8192 ? want : 8192)), block(256);
  hipStream_t s = (hipStream_t)stream;
  const uint8_t *d = (const uint8_t*)dout, *g = (const uint8_t*)gate, *u = (const uint8_t*)up;
  uint8_t *o0 = (uint8_t*)out0, *o1 = (uint8_t*)out1;
#define OMNI_SWIGLU_CASE(DT)                                                                            \
  do {                                                                                                  \
    if (bwd) hipLaunchKernelGGL((swiglu_kernel<DT, true>), grid, block, 0, s, d, g, u, o0, o1, chunks); \
    else hipLaunchKernelGGL((swiglu_kernel<DT, false>), grid, block, 0, s, d, g, u, o0, o1, chunks);    \
  } while (0)
  if (dtype == OMNI_BF16) OMNI_SWIGLU_CASE(kBF16);
  else if (dtype == OMNI_F16) OMNI_SWIGLU_CASE(kF16);
  else OMNI_SWIGLU_CASE(kF32);
#undef OMNI_SWIGLU_CASE
  return to_code(hipGetLastError());
}

extern "C" OMNI_API int32_t omni_swiglu_fwd(const void* gate, const void* up, void* out, int64_t num_elements, int32_t dtype,
                                            void* stream) {
  return swiglu_launch(false, nullptr, gate, up, out, nullptr, num_elements, dtype, stream);
}

extern "C" OMNI_API int32_t omni_swiglu_bwd(const void* dout, const void* gate, const void* up, void* dgate, void* dup,
                                            int64_t num_elements, int32_t dtype, void* stream) {
  return swiglu_launch(true, dout, gate, up, dgate, dup, num_elements, dtype, stream);
}
