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

namespace omni {

// strict "a goes before b": higher score first, then lower payload
__device__ __forceinline__ bool goes_before(float sa, int pa, float sb, int pb) {
  return (sa > sb) || (sa == sb && pa < pb);
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
template <int R, int SIZE>
__device__ __forceinline__ void big_sizes(float (&s)[R], int (&p)[R], const int lane) {
  if constexpr (SIZE <= kWave * R) {
    reg_stages_down<R, SIZE, SIZE / (2 * kWave)>(s, p);
#pragma nounroll
    for (int stride = kWave / 2; stride >= 1; stride >>= 1) lane_stage<R>(s, p, lane, SIZE, stride);
    big_sizes<R, SIZE * 2>(s, p, lane);
  }
}

// Sorts the 64*R (score, payload) items held as item e = reg*64 + lane with a bitonic
// network.  Steps between lanes run as rolled loops (the shuffle distance is a run-time
// value); steps between registers are unrolled so that register indices are constants.
template <int R>
__device__ __forceinline__ void bitonic_sort(float (&s)[R], int (&p)[R], const int lane) {
#pragma nounroll
  for (int size = 2; size <= kWave; size <<= 1) {
#pragma nounroll
    for (int stride = size >> 1; stride >= 1; stride >>= 1) lane_stage<R>(s, p, lane, size, stride);
  }
  big_sizes<R, 2 * kWave>(s, p, lane);
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
constexpr float kNegInf = -__builtin_huge_valf();

// R = half keys per lane (r <= 64*R); C = candidate cells per lane.
template <int R, int C>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_select_kernel(
    const void* __restrict__ lx, const void* __restrict__ ly, void* __restrict__ scores,
    int32_t* __restrict__ indices, int num_tokens, int r, int k, int kp, int dt) {
  const int lane = lane_id();
  const int wave = blockIdx.x * kRouterWaves + (threadIdx.x >> 6);
  const int num_waves = gridDim.x * kRouterWaves;

  // This lane's candidate cells: cell index ci = c*64+lane enumerates rows a = 0..kp-1
  // with min(kp, k/(a+1)) cells each.  Payload (a<<8)|b orders like position a*kp+b.
  int cell[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    int ci = c * kWave + lane, a = 0;
    cell[c] = -1;
    for (; a < kp; ++a) {
      const int cnt = min(kp, k / (a + 1));
      if (ci < cnt) { cell[c] = (a << 8) | ci; break; }
      ci -= cnt;
    }
  }

  for (int t = wave; t < num_tokens; t += num_waves) {
    float sx[R], sy[R];
    int px[R], py[R];
#pragma unroll
    for (int a = 0; a < R; ++a) {
      const int key = a * kWave + lane;
      const bool ok = key < r;
      sx[a] = ok ? load_score(lx, int64_t(t) * r + key, dt) : kNegInf;
      sy[a] = ok ? load_score(ly, int64_t(t) * r + key, dt) : kNegInf;
      px[a] = py[a] = key;
    }
    bitonic_sort<R>(sx, px, lane);
    bitonic_sort<R>(sy, py, lane);

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
        store_score(scores, int64_t(t) * k + j, cs[c], dt);
        indices[int64_t(t) * k + j] = ia * r + ib;
      }
    }
  }
}

static int num_cells(int k, int kp) {
  int n = 0;
  for (int a = 0; a < kp; ++a) n += (kp < k / (a + 1)) ? kp : k / (a + 1);
  return n;
}

template <int R, int C>
static hipError_t launch_select(const void* lx, const void* ly, void* scores, int32_t* indices, int64_t T,
                                int r, int k, int kp, int dt, hipStream_t s) {
  int64_t blocks = (T + kRouterWaves - 1) / kRouterWaves;
  if (blocks > 256 * 16) blocks = 256 * 16;     // waves loop over tokens beyond that
  hipLaunchKernelGGL((router_select_kernel<R, C>), dim3((unsigned)blocks), dim3(kRouterWaves * kWave), 0, s, lx, ly,
                     scores, indices, (int)T, r, k, kp, dt);
  return hipGetLastError();
}

template <int R>
static hipError_t select_by_cells(int cpl, const void* lx, const void* ly, void* scores, int32_t* indices,
                                  int64_t T, int r, int k, int kp, int dt, hipStream_t s) {
  if (cpl <= 1) return launch_select<R, 1>(lx, ly, scores, indices, T, r, k, kp, dt, s);
  if (cpl <= 2) return launch_select<R, 2>(lx, ly, scores, indices, T, r, k, kp, dt, s);
  if (cpl <= 4) return launch_select<R, 4>(lx, ly, scores, indices, T, r, k, kp, dt, s);
  if (cpl <= 8) return launch_select<R, 8>(lx, ly, scores, indices, T, r, k, kp, dt, s);
  return launch_select<R, 16>(lx, ly, scores, indices, T, r, k, kp, dt, s);
}

static int select_dispatch(const void* lx, const void* ly, void* scores, int32_t* indices, int64_t T, int r,
                           int k, int dt, hipStream_t s) {
  const int kp = r < k ? r : k;
  const int cpl = (num_cells(k, kp) + kWave - 1) / kWave;   // <= 11 for k <= 128
  const int rpl = (r + kWave - 1) / kWave;
  hipError_t err;
  if (rpl <= 1) err = select_by_cells<1>(cpl, lx, ly, scores, indices, T, r, k, kp, dt, s);
  else if (rpl <= 2) err = select_by_cells<2>(cpl, lx, ly, scores, indices, T, r, k, kp, dt, s);
  else if (rpl <= 4) err = select_by_cells<4>(cpl, lx, ly, scores, indices, T, r, k, kp, dt, s);
  else if (rpl <= 8) err = select_by_cells<8>(cpl, lx, ly, scores, indices, T, r, k, kp, dt, s);
  else if (rpl <= 16) err = select_by_cells<16>(cpl, lx, ly, scores, indices, T, r, k, kp, dt, s);
  else return OMNI_ERR_UNSUPPORTED;                          // r > 1024
  return err == hipSuccess ? OMNI_OK : OMNI_ERR_HIP_BASE + (int)err;
}

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
  return select_dispatch(logits_x, logits_y, scores, indices, num_tokens, r, k, dtype, (hipStream_t)stream);
}
