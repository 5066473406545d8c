// MFMA GEMMs of the OmniMoE forward path for gfx950 (C = A * B^T, both operands with K
// contiguous, fp32 accumulation on the matrix cores):
//   * router projection   z  = x [Wx;Wy]^T                    (reference omni_moe.py:70-71)
//   * gate/up projection  h  = silu(x Wg^T) * (x Wu^T)         (interface.py:23-29, omni_mlp.py:53-61)
//     - the SwiGLU product is formed in the GEMM epilogue, so gate and up never reach HBM
//   * down projection     y  = h Wd^T (+ expert output)        (interface.py:23-29, omni_moe.py:102)
//
// Structure: a block of 4 waves (2 x 2) owns a (2*TM*32) x (2*TN*32) tile; each wave owns
// TM x TN MFMA tiles of 32x32 and K advances 64 at a time.  The largest tile, 256 x 256, runs
// on 8 waves (2 x 4, two per SIMD) of 128 x 64 instead.  16-bit operands with K % 64 == 0
// take `gemm_nt_dma_kernel` (global -> LDS directly, ring of stages, swizzled rows); anything
// else takes `gemm_nt_kernel` (global -> registers -> one of two LDS stages with padded rows).
// Two more forms of the direct-to-LDS kernel: `gemm_stream_kernel` (the 256 x 256 tile, one block per CU
// walking its output tiles, on 16x16x32 MFMAs) and `gemm_ksplit_kernel` (fewer 64 x 64 tiles than CUs: a
// block's waves share out the K tiles).
// The weight fragment is the MFMA's first operand, so an accumulator lane holds 4 consecutive
// output columns of one row; two lanes pair up to store 8 columns (16 bytes) each.
#include "common.h"
#include "omni_moe_hip.h"

#include <type_traits>

namespace omni {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;                       // K elements per LDS stage
constexpr int kRowBytes = kBK * 2 + 16;       // padded LDS row
constexpr int kGemmThreads = 256;

enum : int { kEpiPlain = 0, kEpiSwiglu = 1, kEpiResidual = 2, kEpiStats = 3, kEpiGate = 4 };   // kEpiStats: plain + column statistics; kEpiGate: silu(acc) * gate, as a pair of 16-bit values

template <int DT> struct ElemBytes { static constexpr int value = (DT == kF32) ? 4 : 2; };

// One 16-byte fragment per lane of each operand: 8 K-values per lane (32x32x16) for 16-bit
// storage; for fp32 the 4 K-values per lane feed four 32x32x2 steps (lane halves pair up
// k and k+4 -- any pairing works as long as both operands use the same one).
template <int DT>
__device__ __forceinline__ f32x16_t mfma32(const u32x4_t a, const u32x4_t b, f32x16_t c) {
  if constexpr (DT == kBF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  } else if constexpr (DT == kF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t ae = a[e], be = b[e];
      c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(ae), __uint_as_float(be), c, 0, 0, 0);
    }
    return c;
  }
}

template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (DT == kBF16) return pack_bf16(lo, hi);
  else if constexpr (DT == kF16) return pack_f16(lo, hi);
  else return 0u;
}

struct GemmArgs {           // all element offsets below are scaled by the element size of DT
  const uint8_t* a;       // [M, K]  activations
  const uint8_t* b0;      // [N, K]  weights (gate weights for SwiGLU)
  const uint8_t* b1;      // [N, K]  up weights (SwiGLU), or the upper half of the columns (plain)
  const uint8_t* res;     // [M, N]  added to the result (residual epilogue only)
  uint8_t* c;             // [M, N]
  int M, N, K;            // N = output columns
  int tiles_m, tiles_n;
  int patch_m, patch_n;   // XCD patch shape (0 = plain order)
  int wide;               // 16-bit output: N % 8 == 0 and C 16-byte aligned, rows are written 16 bytes per lane
  int single;             // N % 4 != 0: rows are not 8-byte aligned, results leave element by element
  float* part_mean;       // kEpiStats only: [ceil(M/32)][N] mean of each column over
  float* part_m2;         //   rows 32s..32s+31 of the ROUNDED result, and the sum of squared deviations
  const float* gate;      // kEpiGate only: [M, N] fp32 factors; C is then [M, 2N]: round(v) in columns 0..N-1, round(v - round(v)) in N..2N-1
  uint8_t* save_gate;     // kEpiSwiglu only, or NULL: [M, N] the rounded gate and up projections, kept for a backward pass
  uint8_t* save_up;       //   (16-byte stores only: N % 8 == 0)
  int exclusive;          // nothing is meant to run beside this launch: the 256 x 256 tile's grid may be one block per CU that holds it to the end
};

// Which output tile a block owns.  Blocks go round-robin over the 8 XCDs; each XCD gets
// compact patches of tiles so that the blocks sharing its L2 share operand panels.
__device__ __forceinline__ void tile_coords(const GemmArgs& g, int& tile_m, int& tile_n) {
  const int b = blockIdx.x;
  if (g.patch_m > 0) {
    const int per_patch = g.patch_m * g.patch_n;
    const int xcd = b & 7, idx = b >> 3;
    const int patch = (idx / per_patch) * 8 + xcd, within = idx % per_patch;
    const int patches_m = g.tiles_m / g.patch_m;
    tile_m = (patch % patches_m) * g.patch_m + within % g.patch_m;
    tile_n = (patch / patches_m) * g.patch_n + within / g.patch_m;
  } else {
    tile_m = b % g.tiles_m;
    tile_n = b / g.tiles_m;
  }
}

// Writes a wave's TM x TN accumulator tiles.  acc[i][j][q] is row m = lane%32 and column
// n = (q/4)*8 + (lane/32)*4 + q%4 of MFMA tile (i, j).
template <int DT, int TM, int TN, int EPI>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& g, f32x16_t (&acc)[TM][TN], const int m0, const int n0,
                                              const int wm, const int wn, const int lane) {
  constexpr int TNO = (EPI == kEpiSwiglu) ? TN / 2 : TN;
  // ---- column statistics of the rounded tile for BatchNorm: every 32-row MFMA tile is one
  // strip.  A column's 32 rows sit in the 32 lanes that share lane/32, one of this lane's 16
  // values each, so the 16 columns of a half-wave are reduced together: a butterfly that halves
  // the values a lane keeps at every step (8 + 4 + 2 + 1 + 1 exchanges) leaves each lane pair
  // with the sum of ONE column; the means travel back the same way (1 + 2 + 4 + 8), the squared
  // deviations are reduced like the sums.  47 register-to-register exchanges per tile.
  if constexpr (EPI == kEpiStats) {
    if (g.part_mean) {
      const bool b16 = lane & 16, b8 = lane & 8, b4 = lane & 4, b2 = lane & 2;
      auto reduce_scatter = [&](const float (&v)[16]) -> float {
        float a8[8], a4[4], a2[2];
#pragma unroll
        for (int e = 0; e < 8; ++e) a8[e] = (b16 ? v[e + 8] : v[e]) + xor_lane_f<16>(b16 ? v[e] : v[e + 8], lane);
#pragma unroll
        for (int e = 0; e < 4; ++e) a4[e] = (b8 ? a8[e + 4] : a8[e]) + xor_lane_f<8>(b8 ? a8[e] : a8[e + 4], lane);
#pragma unroll
        for (int e = 0; e < 2; ++e) a2[e] = (b4 ? a4[e + 2] : a4[e]) + xor_lane_f<4>(b4 ? a4[e] : a4[e + 2], lane);
        const float a1 = (b2 ? a2[1] : a2[0]) + xor_lane_f<2>(b2 ? a2[0] : a2[1], lane);
        return a1 + xor_lane_f<1>(a1, lane);
      };
      // the column this lane ends up with: q = 8*b16 + 4*b8 + 2*b4 + b2
      const int q_mine = (b16 ? 8 : 0) + (b8 ? 4 : 0) + (b4 ? 2 : 0) + (b2 ? 1 : 0);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row0 = m0 + wm * TM * 32 + i * 32;
        const int cnt = min(32, g.M - row0);
        if (cnt <= 0) continue;
        const bool live = (lane & 31) < cnt;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          float v[16];
#pragma unroll
          for (int q = 0; q < 16; ++q) v[q] = live ? Elem<DT>::round(acc[i][j][q]) : 0.f;
          const float mean = reduce_scatter(v) / float(cnt);
          // all-gather of the 16 means, index = column
          float g2[2], g4[4], g8[8], mu[16];
          {
            const float o = xor_lane_f<2>(mean, lane);
            g2[0] = b2 ? o : mean;
            g2[1] = b2 ? mean : o;
          }
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            const float o = xor_lane_f<4>(g2[e], lane);
            g4[e] = b4 ? o : g2[e];
            g4[e + 2] = b4 ? g2[e] : o;
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float o = xor_lane_f<8>(g4[e], lane);
            g8[e] = b8 ? o : g4[e];
            g8[e + 4] = b8 ? g4[e] : o;
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float o = xor_lane_f<16>(g8[e], lane);
            mu[e] = b16 ? o : g8[e];
            mu[e + 8] = b16 ? g8[e] : o;
          }
          float d[16];
#pragma unroll
          for (int q = 0; q < 16; ++q) d[q] = live ? (v[q] - mu[q]) * (v[q] - mu[q]) : 0.f;
          const float m2 = reduce_scatter(d);
          const int n = n0 + wn * TN * 32 + j * 32 + (q_mine >> 2) * 8 + (lane >> 5) * 4 + (q_mine & 3);
          if ((lane & 1) == 0 && n < g.N) {
            g.part_mean[(int64_t)(row0 >> 5) * g.N + n] = mean;
            g.part_m2[(int64_t)(row0 >> 5) * g.N + n] = m2;
          }
        }
      }
    }
  }

  // ---- epilogue.  acc[i][j][q]: row m = lane%32, column n = (q/4)*8 + (lane/32)*4 + q%4
  // value q of column group q4 after the element-wise tail, not yet rounded to storage
  auto value = [&](int i, int j, int q4, int q) -> float {
    if constexpr (EPI == kEpiSwiglu) {
      // the reference materialises gate and up in the storage dtype, then forms
      // silu(gate)*up in fp32 and rounds once (omni_mlp.py:53-61)
      const float gt = Elem<DT>::round(acc[i][j][q4 * 4 + q]);
      const float up = Elem<DT>::round(acc[i][j + TNO][q4 * 4 + q]);
      return (DT == kF32) ? silu_f32(gt) * up : silu_fast(gt) * up;
    } else {
      return acc[i][j][q4 * 4 + q];
    }
  };
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm * TM * 32 + i * 32 + (lane & 31);
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < TNO; ++j) {
      const int nt = n0 + wn * TNO * 32 + j * 32;
      if constexpr (DT != kF32) {
        if (g.wide) {
          // lanes l and l+32 hold columns 8*q4+{0..3} and 8*q4+{4..7} of the same row: one
          // v_permlane32_swap per word regroups two column groups into 8 consecutive columns per
          // lane, so a row receives full 32-byte sectors from every store instruction
#pragma unroll
          for (int pr = 0; pr < 2; ++pr) {
            if (nt + pr * 16 >= g.N) continue;             // same answer in both lanes of a pair
            if constexpr (EPI == kEpiGate) {
              // c = silu(acc) * gate in fp32, stored as a 16-bit head and a 16-bit remainder (head + remainder carries 16
              // significant bits), so that a following GEMM over [head | remainder] sums in nearly full precision
              uint32_t hw[2][2], lw[2][2];
#pragma unroll
              for (int e = 0; e < 2; ++e) {
                const int q4 = 2 * pr + e;
                const int n = nt + q4 * 8 + (lane >> 5) * 4;
                f32x4_t gt = {0.f, 0.f, 0.f, 0.f};
                if (n < g.N) gt = *(const f32x4_t*)(g.gate + (int64_t)m * g.N + n);
                float hv[4], lv[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  const float c = gt[q] != 0.f ? silu_f32(acc[i][j][q4 * 4 + q]) * gt[q] : 0.f;   // an unselected pair contributes exactly 0, whatever its product is
                  hv[q] = Elem<DT>::round(c);
                  lv[q] = c - hv[q];
                }
                hw[e][0] = pack2<DT>(hv[0], hv[1]); hw[e][1] = pack2<DT>(hv[2], hv[3]);
                lw[e][0] = pack2<DT>(lv[0], lv[1]); lw[e][1] = pack2<DT>(lv[2], lv[3]);
              }
              const auto h0 = __builtin_amdgcn_permlane32_swap(hw[0][0], hw[1][0], false, false);
              const auto h1 = __builtin_amdgcn_permlane32_swap(hw[0][1], hw[1][1], false, false);
              const auto l0 = __builtin_amdgcn_permlane32_swap(lw[0][0], lw[1][0], false, false);
              const auto l1 = __builtin_amdgcn_permlane32_swap(lw[0][1], lw[1][1], false, false);
              const int n = nt + pr * 16 + (lane >> 5) * 8;
              if (n < g.N) {
                *(u32x4_t*)(g.c + ((int64_t)m * 2 * g.N + n) * 2) = u32x4_t{h0[0], h1[0], h0[1], h1[1]};
                *(u32x4_t*)(g.c + ((int64_t)m * 2 * g.N + g.N + n) * 2) = u32x4_t{l0[0], l1[0], l0[1], l1[1]};
              }
              continue;
            }
            uint32_t w[2][2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const int q4 = 2 * pr + e;
              float v[4];
#pragma unroll
              for (int q = 0; q < 4; ++q) v[q] = value(i, j, q4, q);
              if constexpr (EPI == kEpiResidual) {
                const int n = nt + q4 * 8 + (lane >> 5) * 4;
                u32x2_t r = {0u, 0u};                      // columns past N are exchanged but never stored
                if (n < g.N) r = *(const u32x2_t*)(g.res + ((int64_t)m * g.N + n) * 2);
                const uint32_t r0 = r[0], r1 = r[1];
                if constexpr (DT == kBF16) {
                  v[0] = Elem<DT>::round(v[0]) + bf16_lo(r0); v[1] = Elem<DT>::round(v[1]) + bf16_hi(r0);
                  v[2] = Elem<DT>::round(v[2]) + bf16_lo(r1); v[3] = Elem<DT>::round(v[3]) + bf16_hi(r1);
                } else {
                  v[0] = Elem<DT>::round(v[0]) + f16_bits_to_f32(r0 & 0xffff); v[1] = Elem<DT>::round(v[1]) + f16_bits_to_f32(r0 >> 16);
                  v[2] = Elem<DT>::round(v[2]) + f16_bits_to_f32(r1 & 0xffff); v[3] = Elem<DT>::round(v[3]) + f16_bits_to_f32(r1 >> 16);
                }
              }
              w[e][0] = pack2<DT>(v[0], v[1]);
              w[e][1] = pack2<DT>(v[2], v[3]);
            }
            const auto s0 = __builtin_amdgcn_permlane32_swap(w[0][0], w[1][0], false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(w[0][1], w[1][1], false, false);
            const int n = nt + pr * 16 + (lane >> 5) * 8;
            if (n < g.N) *(u32x4_t*)(g.c + ((int64_t)m * g.N + n) * 2) = u32x4_t{s0[0], s1[0], s0[1], s1[1]};
            if constexpr (EPI == kEpiSwiglu) {
              if (g.save_gate) {                             // the two rounded projections leave the same way
                uint32_t a[2][2], b[2][2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                  const int q4 = 2 * pr + e;
#pragma unroll
                  for (int h2 = 0; h2 < 2; ++h2) {
                    a[e][h2] = pack2<DT>(acc[i][j][q4 * 4 + 2 * h2], acc[i][j][q4 * 4 + 2 * h2 + 1]);
                    b[e][h2] = pack2<DT>(acc[i][j + TNO][q4 * 4 + 2 * h2], acc[i][j + TNO][q4 * 4 + 2 * h2 + 1]);
                  }
                }
                const auto a0 = __builtin_amdgcn_permlane32_swap(a[0][0], a[1][0], false, false);
                const auto a1 = __builtin_amdgcn_permlane32_swap(a[0][1], a[1][1], false, false);
                const auto b0 = __builtin_amdgcn_permlane32_swap(b[0][0], b[1][0], false, false);
                const auto b1 = __builtin_amdgcn_permlane32_swap(b[0][1], b[1][1], false, false);
                if (n < g.N) {
                  *(u32x4_t*)(g.save_gate + ((int64_t)m * g.N + n) * 2) = u32x4_t{a0[0], a1[0], a0[1], a1[1]};
                  *(u32x4_t*)(g.save_up + ((int64_t)m * g.N + n) * 2) = u32x4_t{b0[0], b1[0], b0[1], b1[1]};
                }
              }
            }
          }
          continue;
        }
      }
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int n = nt + q4 * 8 + (lane >> 5) * 4;
        if (n >= g.N) continue;
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = value(i, j, q4, q);
        if (g.single) {                                  // any N: one element at a time
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if (n + q >= g.N) continue;
            const int64_t at = (int64_t)m * g.N + n + q;
            float out = v[q];
            if constexpr (EPI == kEpiResidual) out = Elem<DT>::round(out) + Elem<DT>::load(g.res, at);
            Elem<DT>::store(g.c, at, out);
          }
          continue;
        }
        const int64_t o = ((int64_t)m * g.N + n) * ElemBytes<DT>::value;   // N is a multiple of 4 here
        if constexpr (EPI == kEpiResidual) {
          // y = round(h Wd^T) + e, rounded again: the reference adds two stored tensors
          if constexpr (DT == kF32) {
            const f32x4_t r = *(const f32x4_t*)(g.res + o);
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] += r[q];
          } else {
            const u32x2_t r = *(const u32x2_t*)(g.res + o);
            const uint32_t r0 = r[0], r1 = r[1];
            if constexpr (DT == kBF16) {
              v[0] = Elem<DT>::round(v[0]) + bf16_lo(r0); v[1] = Elem<DT>::round(v[1]) + bf16_hi(r0);
              v[2] = Elem<DT>::round(v[2]) + bf16_lo(r1); v[3] = Elem<DT>::round(v[3]) + bf16_hi(r1);
            } else {
              v[0] = Elem<DT>::round(v[0]) + f16_bits_to_f32(r0 & 0xffff); v[1] = Elem<DT>::round(v[1]) + f16_bits_to_f32(r0 >> 16);
              v[2] = Elem<DT>::round(v[2]) + f16_bits_to_f32(r1 & 0xffff); v[3] = Elem<DT>::round(v[3]) + f16_bits_to_f32(r1 >> 16);
            }
          }
        }
        if constexpr (DT == kF32) {
          *(f32x4_t*)(g.c + o) = f32x4_t{v[0], v[1], v[2], v[3]};
        } else {
          u32x2_t w = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
          *(u32x2_t*)(g.c + o) = w;
        }
      }
    }
  }
}

// Register-staged kernel, any storage dtype: TM x TN MFMA tiles per wave, K advances by one
// 128-byte row (64 16-bit or 32 fp32 values).  For the SwiGLU epilogue the first TN/2 tiles of
// a wave are gate columns and the last TN/2 the matching up columns.
template <int DT, int TM, int TN, int EPI>
__global__ __launch_bounds__(kGemmThreads, 1) void gemm_nt_kernel(const GemmArgs g) {
  constexpr int BM = 2 * TM * 32;                 // rows of A per block
  constexpr int BR = 2 * TN * 32;                 // rows of the weight tile in LDS per block
  constexpr int BN = (EPI == kEpiSwiglu) ? BR / 2 : BR;   // output columns per block
  constexpr int TNO = (EPI == kEpiSwiglu) ? TN / 2 : TN;  // output tiles per wave along N
  constexpr int kStageBytes = (BM + BR) * kRowBytes;
  extern __shared__ __align__(16) uint8_t lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;

  int tile_m, tile_n;
  tile_coords(g, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // ---- global -> register staging: thread owns 16-byte chunk (tid%8) of rows tid/8 + 32*p
  constexpr int ES = ElemBytes<DT>::value, CE = 16 / ES, BKE = 128 / ES;   // chunk / tile width in elements
  const int ld_chunk = tid & 7, ld_row = tid >> 3;
  constexpr int PA = BM / 32, PB = BR / 32;
  const uint8_t* a_ptr[PA];
  const uint8_t* b_ptr[PB];
#pragma unroll
  for (int p = 0; p < PA; ++p) {
    int row = m0 + p * 32 + ld_row;
    row = row < g.M ? row : g.M - 1;                     // clamp: tail rows are never stored
    a_ptr[p] = g.a + ((int64_t)row * g.K + ld_chunk * CE) * ES;
  }
#pragma unroll
  for (int p = 0; p < PB; ++p) {
    // LDS weight row p*32+ld_row belongs to wave column p/TN, tile p%TN
    const int pw = p / TN, pj = p % TN;
    const uint8_t* base = g.b0;
    int col;
    if constexpr (EPI == kEpiSwiglu) {
      base = (pj < TNO) ? g.b0 : g.b1;
      col = n0 + pw * (TNO * 32) + (pj % TNO) * 32 + ld_row;
    } else {
      col = n0 + p * 32 + ld_row;
    }
    col = col < g.N ? col : g.N - 1;
    if constexpr (EPI == kEpiPlain || EPI == kEpiStats) {
      // optional second weight matrix supplies the upper half of the output columns
      if (g.b1 && col >= g.N / 2) { base = g.b1; col -= g.N / 2; }
    }
    b_ptr[p] = base + ((int64_t)col * g.K + ld_chunk * CE) * ES;
  }
  const int lds_wr = ld_row * kRowBytes + ld_chunk * 16;

  u32x4_t ra[PA], rb[PB];
  auto load_tile = [&](int k0) {
    const bool ok = k0 + ld_chunk * CE < g.K;            // K is a multiple of the chunk: whole chunks
#pragma unroll
    for (int p = 0; p < PA; ++p) ra[p] = ok ? *(const u32x4_t*)(a_ptr[p] + (int64_t)k0 * ES) : u32x4_t{0, 0, 0, 0};
#pragma unroll
    for (int p = 0; p < PB; ++p) rb[p] = ok ? *(const u32x4_t*)(b_ptr[p] + (int64_t)k0 * ES) : u32x4_t{0, 0, 0, 0};
  };
  auto store_tile = [&](int stage) {
    uint8_t* sa = lds + stage * kStageBytes;
    uint8_t* sb = sa + BM * kRowBytes;
#pragma unroll
    for (int p = 0; p < PA; ++p) *(u32x4_t*)(sa + p * 32 * kRowBytes + lds_wr) = ra[p];
#pragma unroll
    for (int p = 0; p < PB; ++p) *(u32x4_t*)(sb + p * 32 * kRowBytes + lds_wr) = rb[p];
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

  // fragment read offsets: lane reads row (lane%32), 16-byte chunk (lane/32) of a 32-byte slab
  const int frag_off = (lane & 31) * kRowBytes + (lane >> 5) * 16;
  const int a_frag = (wm * TM * 32) * kRowBytes + frag_off;
  const int b_frag = BM * kRowBytes + (wn * TN * 32) * kRowBytes + frag_off;

  const int num_kt = (g.K + BKE - 1) / BKE;
  load_tile(0);
  store_tile(0);
  __syncthreads();
  for (int kt = 0; kt < num_kt; ++kt) {
    const uint8_t* st = lds + (kt & 1) * kStageBytes;
    if (kt + 1 < num_kt) load_tile((kt + 1) * BKE);
#pragma unroll
    for (int slab = 0; slab < 4; ++slab) {
      u32x4_t af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = *(const u32x4_t*)(st + a_frag + i * 32 * kRowBytes + slab * 32);
#pragma unroll
      for (int j = 0; j < TN; ++j) bf[j] = *(const u32x4_t*)(st + b_frag + j * 32 * kRowBytes + slab * 32);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = mfma32<DT>(bf[j], af[i], acc[i][j]);
    }
    if (kt + 1 < num_kt) store_tile((kt + 1) & 1);
    __syncthreads();
  }

  gemm_epilogue<DT, TM, TN, EPI>(g, acc, m0, n0, wm, wn, lane);
}

// ---- main kernel: global -> LDS without passing through registers ------------------------
// K advances BK (32 or 64) at a time through a ring of NS LDS stages that
// `global_load_lds_dwordx4` fills directly.  Each wave instruction lands 1 KiB of consecutive
// LDS, so rows cannot be padded; instead the 16-byte chunk c of row r is kept at a swizzled
// chunk position (the loading lane applies the swizzle to its GLOBAL address), chosen so that
// the 128-bit fragment reads of 16 consecutive rows cover all 64 banks once.  NS-2 tiles are
// in flight while one is computed.  The K=16 slabs are skewed across the tile boundary: the
// last slab's fragments of a tile are in registers before the barrier that releases its
// stage, so the MFMAs of one slab always cover the LDS reads of the next.  Needs K % BK == 0.
template <int N> __device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
__device__ __forceinline__ void wait_lds_reads() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// chunk position of logical 16-byte chunk c in row r of a tile whose rows hold BK elements
template <int BK> __device__ __forceinline__ int swizzle(int r, int c) {
  if constexpr (BK == 32) return c ^ ((r >> 2) & 3);      // 4 chunks per 64-byte row
  else return c ^ ((r >> 1) & 7);                          // 8 chunks per 128-byte row
}

template <int DT, int TM, int TN, int EPI, int BK, int NS, int NW = 4>
__global__ __launch_bounds__(NW * 64, 1) void gemm_nt_dma_kernel(const GemmArgs g) {
  // NW waves as 2 (rows) x NW/2 (columns) wave tiles of TM x TN MFMA tiles
  constexpr int BM = 2 * TM * 32, BR = (NW / 2) * TN * 32;
  constexpr int BN = (EPI == kEpiSwiglu) ? BR / 2 : BR;
  constexpr int TNO = (EPI == kEpiSwiglu) ? TN / 2 : TN;
  constexpr int kRow = BK * 2;                         // bytes per LDS row
  constexpr int kCpr = kRow / 16;                      // chunks per row
  constexpr int kRpi = 64 / kCpr;                      // rows one wave instruction fills
  constexpr int kStageBytes = (BM + BR) * kRow;
  constexpr int PA = BM / (NW * kRpi), PB = BR / (NW * kRpi);   // load instructions per wave per tile
  constexpr int LPT = PA + PB;
  constexpr int S = BK / 16;                           // slabs per tile
  extern __shared__ __align__(16) uint8_t lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  int tile_m, tile_n;
  tile_coords(g, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // load instruction p of wave w fills tile rows (4p+w)*kRpi ..: lane -> row lane/kCpr, position lane%kCpr
  const uint8_t* a_src[PA];
  const uint8_t* b_src[PB];
#pragma unroll
  for (int p = 0; p < PA; ++p) {
    const int rl = (NW * p + wave) * kRpi + lane / kCpr;
    const int c = swizzle<BK>(rl, lane % kCpr);        // an involution: position -> logical chunk
    int row = m0 + rl;
    row = row < g.M ? row : g.M - 1;                    // clamp: tail rows are never stored
    a_src[p] = g.a + ((int64_t)row * g.K + c * 8) * 2;
  }
#pragma unroll
  for (int p = 0; p < PB; ++p) {
    const int rl = (NW * p + wave) * kRpi + lane / kCpr;   // row of the weight tile in LDS
    const int c = swizzle<BK>(rl, lane % kCpr);
    const uint8_t* base = g.b0;
    int col;
    if constexpr (EPI == kEpiSwiglu) {
      const int pw = rl / (TN * 32), pj = (rl >> 5) % TN;
      base = (pj < TNO) ? g.b0 : g.b1;
      col = n0 + pw * (TNO * 32) + (pj % TNO) * 32 + (rl & 31);
    } else {
      col = n0 + rl;
    }
    col = col < g.N ? col : g.N - 1;
    if constexpr (EPI == kEpiPlain || EPI == kEpiStats) {
      if (g.b1 && col >= g.N / 2) { base = g.b1; col -= g.N / 2; }
    }
    b_src[p] = base + ((int64_t)col * g.K + c * 8) * 2;
  }

  const int wave_s = __builtin_amdgcn_readfirstlane(wave);   // scalar copy: LDS destinations stay in SGPRs
  // load instruction q (0 .. LPT-1) of tile kt: first the PA instructions of the activation tile, then the weights'
  auto issue_one = [&](int kt, int q) __attribute__((always_inline)) {
    uint8_t* st = lds + (kt % NS) * kStageBytes;
    const int koff = kt * kRow;
    if (q < PA)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a_src[q] + koff),
                                       (__attribute__((address_space(3))) void*)(st + (NW * q + wave_s) * 1024), 16, 0, 0);
    else
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(b_src[q - PA] + koff),
                                       (__attribute__((address_space(3))) void*)(st + BM * kRow + (NW * (q - PA) + wave_s) * 1024), 16, 0, 0);
  };
  auto issue_tile = [&](int kt) {
#pragma unroll
    for (int q = 0; q < LPT; ++q) issue_one(kt, q);
  };

  // fragment reads: lane reads row lane%32, logical chunk 2*slab + lane/32, into buffer slab&1
  const int rl = lane & 31;
  int off_slab[S];
#pragma unroll
  for (int sl = 0; sl < S; ++sl) off_slab[sl] = rl * kRow + swizzle<BK>(rl, 2 * sl + (lane >> 5)) * 16;
  const int a_frag = (wm * TM * 32) * kRow, b_frag = BM * kRow + (wn * TN * 32) * kRow;
  u32x4_t af[2][TM], bf[2][TN];
  // fragment f of a slab: 0 .. TM-1 activation rows, TM .. TM+TN-1 weight rows
  auto read_one = [&](int kt, int slab, int f) __attribute__((always_inline)) {
    const uint8_t* st = lds + (kt % NS) * kStageBytes + off_slab[slab];
    if (f < TM) af[slab & 1][f] = *(const u32x4_t*)(st + a_frag + f * 32 * kRow);
    else bf[slab & 1][f - TM] = *(const u32x4_t*)(st + b_frag + (f - TM) * 32 * kRow);
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

  // One slab = TM*TN MFMAs.  Every MFMA keeps the matrix pipeline busy for 32 cycles, during which
  // this wave may issue other instructions for free -- but a burst of memory instructions takes longer
  // to issue than that and stalls the MFMAs behind it (8 ds_read_b128 in a row cost 9 % of a 16-MFMA
  // slab, one behind each MFMA costs 1 %).  So the memory work of a slab is dealt out behind its MFMAs,
  // a slot each: first the TM + TN fragment reads of the FOLLOWING slab (into the other fragment
  // buffer), then, where a tile is to be fetched, half of that tile's LDS-DMA loads (a tile's loads are
  // issued over two slabs).  The compiler waits for all outstanding LDS reads in front of the next
  // slab's first MFMA; the last read was issued at least TM*TN - (TM+TN) MFMAs earlier.
  constexpr int kMf = TM * TN, kReads = TM + TN, kDmaPerSlab = LPT / 2;
  static_assert(LPT % 2 == 0, "a tile's loads are issued in two halves");
  // kFetch: this slab has slots for loads; they are issued when fetch_kt >= 0 (a scalar branch around
  // each load: control flow around the MFMAs themselves would make the accumulators phi nodes).
  auto slab_step = [&](auto fetch_tag, auto sl_tag, auto next_slab_tag, int next_kt, int fetch_kt, int half) __attribute__((always_inline)) {
    constexpr bool kFetch = decltype(fetch_tag)::value;
    constexpr int sl = decltype(sl_tag)::value, next_slab = decltype(next_slab_tag)::value;
    constexpr int kOps = kReads + (kFetch ? kDmaPerSlab : 0);
    constexpr int kPerSlot = (kOps + kMf - 1) / kMf;
#pragma unroll
    for (int ij = 0; ij < kMf; ++ij) {
      const int i = ij / TN, j = ij % TN;
      acc[i][j] = mfma32<DT>(bf[sl & 1][j], af[sl & 1][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < kPerSlot; ++u) {
        const int op = ij * kPerSlot + u;
        if (op < kReads) read_one(next_kt, next_slab, op);
        else if (kFetch && op < kOps) { if (fetch_kt >= 0) issue_one(fetch_kt, half * kDmaPerSlab + (op - kReads)); }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto slab_then_read = [&](auto sl_tag, auto next_slab_tag, int next_kt) __attribute__((always_inline)) {
    slab_step(std::false_type{}, sl_tag, next_slab_tag, next_kt, -1, 0);
  };
  auto slab_then_read_fetch = [&](auto sl_tag, auto next_slab_tag, int next_kt, int fetch_kt, int half) __attribute__((always_inline)) {
    slab_step(std::true_type{}, sl_tag, next_slab_tag, next_kt, fetch_kt, half);
  };
  // slabs 1 .. S-2 of a tile (no loads are issued during them)
  auto middle_slabs = [&](int kt) __attribute__((always_inline)) {
    if constexpr (S >= 3) slab_then_read(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{}, kt);
    if constexpr (S >= 4) slab_then_read(std::integral_constant<int, 2>{}, std::integral_constant<int, 3>{}, kt);
    static_assert(S <= 4, "at most four slabs per tile");
  };

  const int num_kt = g.K / BK;
#pragma unroll
  for (int t = 0; t < NS; ++t)
    if (t < num_kt) issue_tile(t);
  // before a tile is used, at most NS-2 younger tiles may still be in flight
  auto wait_tile = [&](int younger) {        // younger = tiles issued after the one needed
    if constexpr (NS >= 4) { if (younger >= 2) { wait_vmcnt<2 * LPT>(); return; } }
    if constexpr (NS >= 3) { if (younger >= 1) { wait_vmcnt<LPT>(); return; } }
    wait_vmcnt<0>();
  };
  wait_tile(min(NS, num_kt) - 1 < NS - 2 ? min(NS, num_kt) - 1 : NS - 2);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int f = 0; f < kReads; ++f) read_one(0, 0, f);
  int fetch = -1;                             // tile whose loads are half issued
  for (int kt = 0; kt < num_kt - 1; ++kt) {
    slab_then_read_fetch(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, kt, fetch, 1);   // S >= 2: slab 0 is never the tile's last
    middle_slabs(kt);
    wait_lds_reads();                         // this wave holds every fragment of tile kt
    // tiles kt+1 .. min(kt+NS-1, num_kt-1) are outstanding; tile kt+1 must have landed
    const int younger = num_kt - 2 - kt;
    wait_tile(younger < NS - 2 ? younger : NS - 2);
    __builtin_amdgcn_s_barrier();             // tile kt+1 visible to all; stage of tile kt free
    fetch = (kt + NS < num_kt) ? kt + NS : -1;
    __builtin_amdgcn_sched_barrier(0);
    slab_then_read_fetch(std::integral_constant<int, S - 1>{}, std::integral_constant<int, 0>{}, kt + 1, fetch, 0);
  }
  slab_then_read(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, num_kt - 1);   // last tile
  middle_slabs(num_kt - 1);
#pragma unroll
  for (int ij = 0; ij < kMf; ++ij) acc[ij / TN][ij % TN] = mfma32<DT>(bf[(S - 1) & 1][ij % TN], af[(S - 1) & 1][ij / TN], acc[ij / TN][ij % TN]);
  gemm_epilogue<DT, TM, TN, EPI>(g, acc, m0, n0, wm, wn, lane);
}

// ---- the 256 x 256 tile as a stream over several output tiles ----------------------------------------
// One block per CU walks its share of the output tiles (tile index blockIdx, blockIdx + gridDim, ...).  The K tiles of
// consecutive output tiles form ONE stream through the two LDS stages: while a block multiplies the last K tiles of an
// output tile, the first K tiles of its next one are already on their way, so only a block's first output tile waits for
// memory before its first matrix instruction.  Ring loads are buffer loads (scalar base and tile offsets, one 32-bit
// lane offset per operand).  The grid keeps every CU until the kernel ends, so a kernel on another stream finds no room
// beside it: the callers use this form where nothing is meant to run concurrently.
// Needs N a multiple of the tile's columns and K % 64 == 0; a ragged last row tile re-reads the matrix's last row and stores
// nothing for it.  XCD patches need whole rounds of 256 tiles; other tile counts go in plain order.
//
// The wave's 128 x 64 tile is 8 x 4 MFMA tiles of 16 x 16 and K advances 32 per instruction.  Under sustained load the
// board clocks by power, and on the same operand bits the 16 x 16 x 32 instruction sustains about 15 % more than
// 32 x 32 x 16 (register-only probes, two waves per SIMD: 2.07 against 1.80 PFLOP/s; this kernel against the same
// kernel on 32 x 32 x 16: 8192 x 8192 x 2048 207 against 222 us, 32768 x 2 x 8192 x 2048 with SwiGLU 1.66 against
// 1.76 ms, 4096 x 2 x 4096 x 1024 level).  A lane of accumulator tile (i, j) holds row m = 16 i + lane%16 and the four
// columns n = 16 j + 4 (lane/16) + 0..3.  The activation fragments are a single set that is refilled row by row (the
// fragment of row tile i for the next K step is read as soon as row i's four instructions have issued); the weight
// fragments alternate between two sets.
__device__ __forceinline__ void tile_coords_of(const GemmArgs& g, int b, int& tile_m, int& tile_n) {
  if (g.patch_m > 0) {
    const int per_patch = g.patch_m * g.patch_n;
    const int xcd = b & 7, idx = b >> 3;
    const int patch = (idx / per_patch) * 8 + xcd, within = idx % per_patch;
    const int patches_m = g.tiles_m / g.patch_m;
    tile_m = (patch % patches_m) * g.patch_m + within % g.patch_m;
    tile_n = (patch / patches_m) * g.patch_n + within / g.patch_m;
  } else {
    tile_m = b % g.tiles_m;
    tile_n = b / g.tiles_m;
  }
}

template <int DT>
__device__ __forceinline__ f32x4_t mfma16(const u32x4_t a, const u32x4_t b, f32x4_t c) {
  if constexpr (DT == kBF16) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// Epilogue of the streaming kernel (full column tiles, 16-byte stores; rows past M are not stored).  Lanes l and l ^ 16 hold columns 4g..4g+3 and 4g+4..4g+7 of
// two neighbouring column tiles: one v_permlane16_swap per word leaves every lane with 8 consecutive columns of one
// of the two tiles, 64 consecutive bytes of a row over the four lanes l, l + 16, l + 32, l + 48.  The store path wants
// those four in CONSECUTIVE lanes: a store-only microbenchmark moves 14 bytes per cycle and CU when neighbouring lanes
// write different rows (16 rows x 64 bytes or 8 rows x 128 bytes per instruction alike) and 26-27 when each quad of
// lanes writes 64 bytes on end, in any order of its four pieces; and while a tile's stores pass through that path the
// ring loads of the next tile queue behind them.  So every word goes through one ds_bpermute_b32 (lane d takes from
// lane d / 4 + 16 (d % 4); no LDS memory involved), after which lane d holds 16 bytes of row d / 4.  The residual is
// fetched in that layout as well, 16 bytes per lane, and added to the rounded product there: the same arithmetic.
__device__ __forceinline__ u32x4_t to_row_quads(const uint32_t x0, const uint32_t x1, const uint32_t x2, const uint32_t x3, const int from) {
  return u32x4_t{(uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)x0), (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)x1),
                 (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)x2), (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)x3)};
}
template <int DT> __device__ __forceinline__ float half_lo(const uint32_t w) {
  if constexpr (DT == kBF16) return bf16_lo(w); else return f16_bits_to_f32((uint16_t)(w & 0xffffu));
}
template <int DT> __device__ __forceinline__ float half_hi(const uint32_t w) {
  if constexpr (DT == kBF16) return bf16_hi(w); else return f16_bits_to_f32((uint16_t)(w >> 16));
}
template <int DT, int EPI>
__device__ __forceinline__ void stream_epilogue(const GemmArgs& g, f32x4_t (&acc)[8][4], const int m0, const int n0, const int wm,
                                                  const int wn, const int lane) {
  constexpr int TNO = (EPI == kEpiSwiglu) ? 2 : 4;
  const int nb = n0 + wn * (TNO * 16);
  // (not for the SwiGLU form, whose epilogue is bound by its arithmetic: there the exchange costs the layer step 0.4 %)
  constexpr bool kQuads = EPI != kEpiSwiglu;
  const int tr = kQuads ? lane >> 2 : lane & 15;       // where the lane's 16 bytes go: row of the 16,
  const int tg = kQuads ? lane & 3 : lane >> 4;        // ... piece of the row's 64 bytes
  const int from = (tr + 16 * tg) * 4;                 // ds_bpermute address of the lane that holds them before the exchange
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = m0 + wm * 128 + i * 16 + tr;
    const bool stored = m < g.M;
#pragma unroll
    for (int j = 0; j < TNO; j += 2) {
      uint32_t w[2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if constexpr (EPI == kEpiSwiglu) {
            // gate and up are materialised in the storage dtype, silu(gate)*up is formed in fp32 and rounded once (omni_mlp.py:53-61)
            const float gt = Elem<DT>::round(acc[i][j + t][q]), up = Elem<DT>::round(acc[i][j + t + TNO][q]);
            v[q] = silu_fast(gt) * up;
          } else {
            v[q] = acc[i][j + t][q];
          }
        }
        w[t][0] = pack2<DT>(v[0], v[1]);
        w[t][1] = pack2<DT>(v[2], v[3]);
      }
      // odd 16-lane rows of tile j's words change places with even rows of tile j+1's
      const auto s0 = __builtin_amdgcn_permlane16_swap(w[0][0], w[1][0], false, false);
      const auto s1 = __builtin_amdgcn_permlane16_swap(w[0][1], w[1][1], false, false);
      u32x4_t out = kQuads ? to_row_quads(s0[0], s1[0], s0[1], s1[1], from) : u32x4_t{s0[0], s1[0], s0[1], s1[1]};
      const int n = nb + (j + (tg & 1)) * 16 + (tg & 2) * 4;
      const int64_t at = ((int64_t)m * g.N + n) * 2;
      if constexpr (EPI == kEpiResidual) {
        const int mr = stored ? m : g.M - 1;             // rows past the matrix are computed but never stored
        const u32x4_t r = *(const u32x4_t*)(g.res + ((int64_t)mr * g.N + n) * 2);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t o = out[q], rq = r[q];
          out[q] = pack2<DT>(half_lo<DT>(o) + half_lo<DT>(rq), half_hi<DT>(o) + half_hi<DT>(rq));
        }
      }
      if (stored) *(u32x4_t*)(g.c + at) = out;
      if constexpr (EPI == kEpiSwiglu) {
        if (g.save_gate) {                               // the two rounded projections leave the same way (kept for a backward pass)
          uint32_t a[2][2], b[2][2];
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
              a[t][h2] = pack2<DT>(acc[i][j + t][2 * h2], acc[i][j + t][2 * h2 + 1]);
              b[t][h2] = pack2<DT>(acc[i][j + t + TNO][2 * h2], acc[i][j + t + TNO][2 * h2 + 1]);
            }
          const auto a0 = __builtin_amdgcn_permlane16_swap(a[0][0], a[1][0], false, false);
          const auto a1 = __builtin_amdgcn_permlane16_swap(a[0][1], a[1][1], false, false);
          const auto b0 = __builtin_amdgcn_permlane16_swap(b[0][0], b[1][0], false, false);
          const auto b1 = __builtin_amdgcn_permlane16_swap(b[0][1], b[1][1], false, false);
          const u32x4_t ga = {a0[0], a1[0], a0[1], a1[1]}, ub = {b0[0], b1[0], b0[1], b1[1]};
          if (stored) {
            *(u32x4_t*)(g.save_gate + at) = ga;
            *(u32x4_t*)(g.save_up + at) = ub;
          }
        }
      }
    }
  }
}

template <int DT, int EPI>
__global__ __launch_bounds__(512, 1) void gemm_stream_kernel(const GemmArgs g) {
  constexpr int TM = 8, TN = 4;                      // MFMA tiles of 16 x 16 per wave: 128 x 64
  constexpr int BM = 256, BR = 256;
  constexpr int BN = (EPI == kEpiSwiglu) ? 128 : 256;
  constexpr int kRow = 128, kStage = (BM + BR) * kRow;
  extern __shared__ __align__(16) uint8_t lds[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const int num_kt = g.K / 64;
  const int num_tiles = g.tiles_m * g.tiles_n;
  const uint32_t row_bytes = (uint32_t)g.K * 2;

  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void*)g.a, 0, 0x7fffffff, 0x00020000);
  const uint8_t* bsel = (EPI == kEpiSwiglu && (wave >> 2)) ? g.b1 : g.b0;      // waves 0-3 fetch gate rows, 4-7 the up rows
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void*)bsel, 0, 0x7fffffff, 0x00020000);
  // plain and residual forms: an optional second weight matrix supplies the upper half of the output columns (whole tiles of it)
  const __amdgpu_buffer_rsrc_t rsrc_hi = __builtin_amdgcn_make_buffer_rsrc((void*)((EPI != kEpiSwiglu && g.b1) ? g.b1 : g.b0), 0, 0x7fffffff, 0x00020000);

  // Load instruction p of a wave fills LDS rows (8p + wave)*8 + lane/8 of a tile; the lane fetches the logical chunk that
  // belongs at its (swizzled) position, which depends on the wave's parity and the lane only.  For the SwiGLU form rows
  // 64p .. 64p+31 of the weight tile are gate rows and 64p+32 .. 64p+63 the matching up rows of wave column p.
  const int sw = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
  uint32_t a_voff[4];                                  // per load instruction: its row of the tile, clamped to the matrix (set with the cursor)
  const uint32_t b_voff = (uint32_t)((EPI == kEpiSwiglu ? (wave & 3) * 8 : wave * 8) + (lane >> 3)) * row_bytes + sw * 16;
  constexpr int kBRowsPerInstr = (EPI == kEpiSwiglu) ? 32 : 64;     // weight rows between consecutive load instructions of a wave

  uint32_t b_voff4[4];                                 // ... and per weight load instruction of the wave
#pragma unroll
  for (int q = 0; q < 4; ++q) b_voff4[q] = b_voff + (uint32_t)(q * kBRowsPerInstr) * row_bytes;

  // Fetch cursor: the next K tile of the stream to request.  Everything a load instruction needs beyond its lane offsets is
  // kept ready in scalar registers and moved on once per K tile (the K loop otherwise spends four scalar instructions
  // on every matrix instruction, and a wave issues in order): the LDS address of the wave's first row in the cursor's
  // stage, the byte offset of the K tile within the activation and the weight rows, the weight matrix's descriptor.
  using LdsPtr = __attribute__((address_space(3))) void*;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(LdsPtr)lds;
  int f_tile = blockIdx.x, f_kt = 0;
  uint32_t f_ldsw = lds_base + (uint32_t)wave * 1024;  // ... of the wave's first row in the cursor's stage
  int f_flip = kStage;                                 // to the other stage and back
  uint32_t f_sa = 0, f_sb = 0;
  int half_pending = 0;                                // the cursor's K tile has its activation half requested, not yet its weights (an int: a bool carried round the loop becomes a lane mask)
  __amdgpu_buffer_rsrc_t rsrc_w = rsrc_b;              // the second weight matrix for the upper half of the columns (plain and residual forms)
  auto cursor_coords = [&]() {                         // at a tile's first K tile
    int tm, tn;
    tile_coords_of(g, f_tile, tm, tn);
    f_sa = (uint32_t)(tm * BM) * row_bytes;
    const bool hi = EPI != kEpiSwiglu && g.b1 != nullptr && tn * BN >= g.N / 2;
    rsrc_w = hi ? rsrc_hi : rsrc_b;
    f_sb = (uint32_t)(tn * BN - (hi ? g.N / 2 : 0)) * row_bytes;
    const int last = g.M - 1 - tm * BM;                // last row of the matrix, counted from the tile's first: a ragged last tile re-reads it
#pragma unroll
    for (int q = 0; q < 4; ++q) a_voff[q] = (uint32_t)min(q * 64 + wave * 8 + (lane >> 3), last) * row_bytes + sw * 16;
  };
  cursor_coords();
  auto issue_one = [&](int q) __attribute__((always_inline)) {       // q = 0..3: activation rows, 4..7: weight rows
    if (q < 4)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (LdsPtr)(uintptr_t)(f_ldsw + q * 8192), 16, a_voff[q], f_sa, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (LdsPtr)(uintptr_t)(f_ldsw + BM * kRow + (q - 4) * 8192), 16, b_voff4[q - 4], f_sb, 0, 0);
  };
  auto cursor_advance = [&]() {                        // after a K tile's second half has been issued
    f_ldsw += (uint32_t)f_flip;
    f_flip = -f_flip;
    if (++f_kt == num_kt) {
      f_kt = 0;
      f_tile += gridDim.x;
      if (f_tile < num_tiles) cursor_coords();
    } else {
      f_sa += 128;
      f_sb += 128;
    }
  };

  // fragment reads: lane reads row lane%16 of a 16-row tile, logical chunk 4*kstep + lane/16 (8 K values of the step's 32).
  // ra[1], rb[1]: the lane's activation / weight fragment row of K step 1 in the stage being multiplied; ra[0], rb[0]: of K step 0
  // in the OTHER stage (the next K tile's) -- what the first and the second step of a K tile read for the step after them;
  // the row tile comes as the instruction's immediate offset, and the four change stages once per K tile (c_flip).
  const int r16 = lane & 15;
  uint32_t ra[2], rb[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const uint32_t off = lds_base + (uint32_t)(r16 * kRow + ((4 * ks + (lane >> 4)) ^ (r16 >> 1)) * 16) + (ks == 0 ? (uint32_t)kStage : 0u);
    ra[ks] = (uint32_t)((wm * 128) * kRow) + off;
    rb[ks] = (uint32_t)(BM * kRow + (wn * 64) * kRow) + off;
  }
  int c_flip[2] = {-kStage, kStage};                   // next change of ra[ks], rb[ks]
  using LdsFrag = const __attribute__((address_space(3))) u32x4_t*;
  u32x4_t af[TM], bf[2][TN];
  auto read_a = [&](int ks, int i) __attribute__((always_inline)) { af[i] = *(LdsFrag)(uintptr_t)(ra[ks] + i * 16 * kRow); };
  auto read_b = [&](int ks, int j) __attribute__((always_inline)) { bf[ks][j] = *(LdsFrag)(uintptr_t)(rb[ks] + j * 16 * kRow); };

  f32x4_t acc[TM][TN];
  auto clear_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[i][j][q] = 0.f;
  };
  clear_acc();

  constexpr int kEpiStores = (EPI == kEpiSwiglu) ? 8 : 16;   // store instructions of a wave's epilogue (no memory instruction follows them)
  // One K step of 32: TM*TN matrix instructions in row order, at most one memory instruction behind each (slot_op).
  // In the K tile's second step, whose following step reads the other stage, the wave waits after row 0 for its fragment
  // reads and ring loads and meets the block.
  constexpr int kSyncRow = 0;
  // what follows matrix instruction (i, j): 0 nothing, 10+n weight fragment n, 20+n activation fragment n of the following
  // step, 30+n ring load n of the cursor's K tile (0-3 activation rows, in the second step; 4-7 weight rows, in the first)
  auto slot_op = [](bool second, int i, int j) constexpr -> int {
    if (j == 0 && i >= 1 && i <= 4) return 10 + (i - 1);
    if (j == 1 && i >= 1 && i <= 4) return second ? 30 + (i - 1) : 34 + (i - 1);
    if (second && j == 1 && i >= 5) return 40 + (i - 5);            // 40-43: the weight rows too, in a tile's last K tile
    if (second && j == 2 && i == 7) return 43;
    if (j == 2 && i == 1) return 20;
    if (j == 3 && i >= 1) return 20 + i;
    return 0;
  };
  // last: the output tile's last K tile; young: memory instructions of the wave issued after the loads this K tile's sync
  // point waits for (the previous tile's stores, when the K tile is a tile's first)
  auto kstep = [&](auto ks_tag, auto sync_tag, const int last, const int young) __attribute__((always_inline)) {
    constexpr int ks = decltype(ks_tag)::value;
    constexpr bool sync = decltype(sync_tag)::value;
    constexpr int nks = ks ^ 1;
    // (scalar registers by force: left alone the compiler keeps these loop-carried flags in vector registers and tests them there)
    const bool fa = f_tile < num_tiles;
    const bool hp = half_pending != 0;
    const bool fl = fa && last;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc[i][j] = mfma16<DT>(bf[ks][j], af[i], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
        const int op = slot_op(sync, i, j);
        if (op >= 10 && op < 20) read_b(nks, op - 10);
        if (op >= 20 && op < 30) read_a(nks, op - 20);
        if (op >= 30 && op < 34) { if (fa) issue_one(op - 30); }
        if (op >= 34 && op < 40) { if (hp) issue_one(op - 30); }
        if (op >= 40) { if (fl) issue_one(op - 36); }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (sync) {
        if (i == kSyncRow) {
          wait_lds_reads();                            // this wave holds every fragment of the K tile
          // the next K tile has landed.  The counter runs in issue order, loads and stores alike: behind a tile's epilogue
          // its stores are younger than every load of the next K tile (whose weight rows a tile's last K tile requests
          // early for that reason) and may stay in flight for another K tile
          if (young == kEpiStores) wait_vmcnt<kEpiStores>(); else wait_vmcnt<0>();
          __builtin_amdgcn_s_barrier();                // ... for all waves; this K tile's stage is free
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
  auto k_tile = [&](const int last, const int young) __attribute__((always_inline)) {
    kstep(I0{}, std::false_type{}, last, 0);           // the weights of the K tile whose activations were requested one step ago
    if (half_pending) { cursor_advance(); half_pending = 0; }
    const int fa = f_tile < num_tiles ? 1 : 0;
    kstep(I1{}, std::true_type{}, last, young);        // the activations of the K tile two ahead go into the freed stage
    if (last & fa) cursor_advance();                   // ... with its weights, when the epilogue comes next
    half_pending = fa & (last ^ 1);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) { ra[ks] += (uint32_t)c_flip[ks]; rb[ks] += (uint32_t)c_flip[ks]; c_flip[ks] = -c_flip[ks]; }
  };

  // ---- prologue: the stream's first two K tiles
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int q = 0; q < 8; ++q) issue_one(q);
    cursor_advance();
  }
  wait_vmcnt<8>();                                     // the first K tile has landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < TM; ++i) af[i] = *(LdsFrag)(uintptr_t)(ra[0] - (uint32_t)kStage + i * 16 * kRow);     // K step 0 of stage 0
#pragma unroll
  for (int j = 0; j < TN; ++j) bf[0][j] = *(LdsFrag)(uintptr_t)(rb[0] - (uint32_t)kStage + j * 16 * kRow);

  int young = 0;                                       // stores of the previous tile's epilogue, if their number is known
  for (int tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    // (not unrolled, which would include peeling the first K tile off as a second loop body: the compiler then gives the
    // accumulators different registers in the two bodies and the kernel needs 250 VGPRs instead of 216, which leaves no
    // room on a SIMD for a wave of the kernels that the layer runs beside this one)
#pragma clang loop unroll(disable)
    for (int kt = 0; kt < num_kt; ++kt) k_tile(kt == num_kt - 1 ? 1 : 0, kt == 0 ? young : 0);
    int tm, tn;
    tile_coords_of(g, tile, tm, tn);
    stream_epilogue<DT, EPI>(g, acc, tm * BM, tn * BN, wm, wn, lane);
    // every row of the wave inside the matrix: each store instruction of the epilogue has been issued
    young = (g.M - tm * BM - wm * 128 >= 128 && !(EPI == kEpiSwiglu && g.save_gate)) ? kEpiStores : 0;
    clear_acc();
  }
}

// ---- few output tiles, long K: the K tiles of one 64 x 64 output tile dealt out over the block's four waves ----------
// A product like the router projection at a few thousand tokens (4096 x 128 x 1024) has too few output tiles to fill the
// GPU and its time is the latency of one block's K loop: with the ring kernel above, 16 rounds of wait - barrier - four
// MFMAs.  Here every wave multiplies the whole 64 x 64 tile (2 x 2 MFMA tiles) over ITS K tiles (kt = wave, wave + 4,
// ...) through a two-stage LDS ring of its own, so the K loop is a quarter as long, has four independent accumulators
// to keep the matrix pipeline fed, and meets no block barrier: a wave waits only for its own loads.  The four partial
// tiles then meet in LDS (summed in wave order, so the result does not depend on timing), and wave w finishes MFMA tile
// (w % 2, w / 2) with the common epilogue.  Needs K % 64 == 0; worth it while there are fewer tiles than CUs.
template <int DT, int EPI>
__global__ __launch_bounds__(kGemmThreads, 1) void gemm_ksplit_kernel(const GemmArgs g) {
  constexpr int kRow = 128, kTile = 64 * kRow;          // one operand's 64 rows of a K tile
  constexpr int kStage = 2 * kTile, kRing = 2 * kStage; // per wave: two stages of [activations | weights]
  extern __shared__ __align__(16) uint8_t lds[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tile_m = blockIdx.x % g.tiles_m, tile_n = blockIdx.x / g.tiles_m;
  const int m0 = tile_m * 64, n0 = tile_n * 64;
  uint8_t* ring = lds + wave * kRing;

  // load instruction p (0..7) fills rows 8p + lane/8 of an operand tile; the lane fetches the logical chunk that belongs at
  // its (swizzled) position
  const uint8_t* a_src[8];
  const uint8_t* b_src[8];
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const int rl = p * 8 + (lane >> 3);
    const int c = swizzle<64>(rl, lane & 7);
    int row = m0 + rl;
    row = row < g.M ? row : g.M - 1;                    // clamp: tail rows and columns are never stored
    a_src[p] = g.a + ((int64_t)row * g.K + c * 8) * 2;
    int col = n0 + rl;
    col = col < g.N ? col : g.N - 1;
    const uint8_t* base = g.b0;
    if constexpr (EPI == kEpiPlain || EPI == kEpiStats) {
      if (g.b1 && col >= g.N / 2) { base = g.b1; col -= g.N / 2; }
    }
    b_src[p] = base + ((int64_t)col * g.K + c * 8) * 2;
  }
  auto issue_tile = [&](int kt, int stage) __attribute__((always_inline)) {
    uint8_t* st = ring + stage * kStage;
    const int koff = kt * kRow;
#pragma unroll
    for (int p = 0; p < 8; ++p)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a_src[p] + koff),
                                       (__attribute__((address_space(3))) void*)(st + p * 1024), 16, 0, 0);
#pragma unroll
    for (int p = 0; p < 8; ++p)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(b_src[p] + koff),
                                       (__attribute__((address_space(3))) void*)(st + kTile + p * 1024), 16, 0, 0);
  };

  // fragment reads: lane reads row lane%32 (+32 i), logical chunk 2*slab + lane/32
  const int rl = lane & 31;
  int off_slab[4];
#pragma unroll
  for (int sl = 0; sl < 4; ++sl) off_slab[sl] = rl * kRow + swizzle<64>(rl, 2 * sl + (lane >> 5)) * 16;

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

  const int num_kt = g.K / 64;
  const int mine = (num_kt - wave + 3) / 4;             // K tiles wave, wave + 4, ...
  if (mine > 0) issue_tile(wave, 0);
  if (mine > 1) issue_tile(wave + 4, 1);
  for (int t = 0; t < mine; ++t) {
    if (t + 1 < mine) wait_vmcnt<16>(); else wait_vmcnt<0>();     // this tile has landed; the next one may be in flight
    const uint8_t* st = ring + (t & 1) * kStage;
    u32x4_t af[2][2], bf[2][2];
    auto read_slab = [&](int sl) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < 2; ++i) af[sl & 1][i] = *(const u32x4_t*)(st + off_slab[sl] + i * 32 * kRow);
#pragma unroll
      for (int j = 0; j < 2; ++j) bf[sl & 1][j] = *(const u32x4_t*)(st + kTile + off_slab[sl] + j * 32 * kRow);
    };
    read_slab(0);
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      if (sl + 1 < 4) read_slab(sl + 1);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma32<DT>(bf[sl & 1][j], af[sl & 1][i], acc[i][j]);
    }
    if (t + 2 < mine) {
      wait_lds_reads();                                  // the stage is read out (by this wave, its only reader)
      issue_tile(wave + 4 * (t + 2), t & 1);
    }
  }

  // ---- the four partial tiles meet in LDS: [wave][MFMA tile][column group][lane] 16 bytes each
  __syncthreads();                                       // every wave is done with its ring
  f32x4_t* xch = (f32x4_t*)lds;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        xch[((wave * 4 + (j * 2 + i)) * 4 + q4) * 64 + lane] =
            f32x4_t{acc[i][j][q4 * 4], acc[i][j][q4 * 4 + 1], acc[i][j][q4 * 4 + 2], acc[i][j][q4 * 4 + 3]};
  __syncthreads();
  f32x16_t sum[1][1];
#pragma unroll
  for (int q4 = 0; q4 < 4; ++q4) {
    f32x4_t v = xch[((0 * 4 + wave) * 4 + q4) * 64 + lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const f32x4_t o = xch[((w * 4 + wave) * 4 + q4) * 64 + lane];
      v[0] += o[0]; v[1] += o[1]; v[2] += o[2]; v[3] += o[3];
    }
    sum[0][0][q4 * 4] = v[0]; sum[0][0][q4 * 4 + 1] = v[1]; sum[0][0][q4 * 4 + 2] = v[2]; sum[0][0][q4 * 4 + 3] = v[3];
  }
  gemm_epilogue<DT, 1, 1, EPI>(g, sum, m0, n0, wave & 1, wave >> 1, lane);
}

// One list entry per kernel instantiation that launch_gemm can start (the static members come into being
// at library load for every instantiation the dispatch below names).
template <int DT, int TM, int TN, int EPI, int BK, int NS, int NW = 4>
struct DmaKernelLds {
  static inline LdsKernel entry{(const void*)gemm_nt_dma_kernel<DT, TM, TN, EPI, BK, NS, NW>, NS * (2 * TM * 32 + (NW / 2) * TN * 32) * BK * 2};
};
template <int DT, int EPI>
struct StreamKernelLds {
  static inline LdsKernel entry{(const void*)gemm_stream_kernel<DT, EPI>, 2 * 512 * 128};
};
template <int DT, int EPI>
struct KsplitKernelLds {
  static inline LdsKernel entry{(const void*)gemm_ksplit_kernel<DT, EPI>, 4 * 2 * 2 * 64 * 128};
};
template <int DT, int TM, int TN, int EPI>
struct StagedKernelLds {
  static inline LdsKernel entry{(const void*)gemm_nt_kernel<DT, TM, TN, EPI>, 2 * (2 * TM * 32 + 2 * TN * 32) * kRowBytes};
};

template <int DT, int TM, int TN, int EPI>
static hipError_t launch_gemm(GemmArgs g, hipStream_t s) {
  constexpr int BM = 2 * TM * 32, BR = 2 * TN * 32, BN = (EPI == kEpiSwiglu) ? BR / 2 : BR;
  constexpr int kLds = 2 * (BM + BR) * kRowBytes;
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + BN - 1) / BN;
  const int blocks = g.tiles_m * g.tiles_n;
  // one XCD runs 32 blocks at a time: give it 4 x 8 patches when the tile grid allows
  g.patch_m = g.patch_n = 0;
  g.wide = (DT != kF32) && g.N % 8 == 0 && ((uintptr_t)g.c % 16 == 0);
  g.single = g.N % 4 != 0;
  if (EPI == kEpiGate && !(g.wide && (uintptr_t)g.gate % 16 == 0)) return hipErrorInvalidValue;   // the gate epilogue has the 16-byte form only
  if (EPI == kEpiSwiglu && g.save_gate && !g.wide) return hipErrorInvalidValue;                  // so has the saving SwiGLU epilogue
  if (blocks % 256 == 0) {
    if (g.tiles_m % 4 == 0 && g.tiles_n % 8 == 0) { g.patch_m = 4; g.patch_n = 8; }
    else if (g.tiles_m % 8 == 0 && g.tiles_n % 4 == 0) { g.patch_m = 8; g.patch_n = 4; }
  }
  // 128-byte LDS rows (64-byte rows halve the fetch rate); as many ring stages as 160 KiB hold, up to 4
  constexpr int kDmaBK = 64;
  constexpr int kFit = (160 * 1024) / ((BM + BR) * kDmaBK * 2);
  constexpr int kDmaStages = kFit > 4 ? 4 : kFit;
  if constexpr (DT != kF32) if (g.K % kDmaBK == 0) {
    constexpr int kDmaLds = kDmaStages * (BM + BR) * kDmaBK * 2;
    static_assert(kDmaLds <= 160 * 1024, "LDS ring exceeds 160 KiB");
    if constexpr (TM == 4 && TN == 4 && (EPI == kEpiPlain || EPI == kEpiSwiglu || EPI == kEpiResidual)) {
      // full column tiles, K tiles enough for the two-stage prologue (buffer loads: operands below 1 Gi elements, 16-byte
      // aligned).  Nothing meant to run beside it: one block per CU streams through its tiles.  Otherwise the same kernel
      // with one block per tile, so that CUs come free for the other stream's kernels as blocks retire (two-stream layer
      // step at 4096 tokens, 1024 x 4096: 123.3 us against 127.2 us with the 32x32x16 kernel below in that place).
      const bool covers = g.N % BN == 0 && g.K >= 2 * kDmaBK && blocks >= 256 && g.wide &&
                          (EPI == kEpiSwiglu || !g.b1 || (g.N / 2) % BN == 0) && (int64_t)g.M * g.K < (1ll << 30) &&
                          (int64_t)g.N * g.K < (1ll << 30) && (uintptr_t)g.a % 16 == 0 && (uintptr_t)g.b0 % 16 == 0 &&
                          (!g.b1 || (uintptr_t)g.b1 % 16 == 0);
      if (covers) {
        if (hipError_t e = StreamKernelLds<DT, EPI>::entry.ensure(); e != hipSuccess) return e;
        hipLaunchKernelGGL((gemm_stream_kernel<DT, EPI>), dim3(g.exclusive ? 256 : blocks), dim3(512), 2 * 512 * 128, s, g);
        return hipGetLastError();
      }
    }
    if constexpr (TM == 1 && TN == 1 && EPI != kEpiSwiglu && EPI != kEpiGate) {
      // fewer 64 x 64 tiles than CUs and at least two K tiles per wave: the K tiles dealt out over the waves
      if (blocks <= 256 && g.K >= 512) {
        if (hipError_t e = KsplitKernelLds<DT, EPI>::entry.ensure(); e != hipSuccess) return e;
        hipLaunchKernelGGL((gemm_ksplit_kernel<DT, EPI>), dim3(blocks), dim3(kGemmThreads), 4 * 2 * 2 * 64 * 128, s, g);
        return hipGetLastError();
      }
    }
    if constexpr (TM == 4 && TN == 4) {
      // the 256 x 256 block tile on 8 waves of 128 x 64, two per SIMD: one wave's barrier and load waits are the other's
      // issue slots (gate/up projection at 4096 x 4096 x 1024: 66.7 against 69.1 us), at 6 fragment reads per 8 MFMAs
      auto kern8 = gemm_nt_dma_kernel<DT, 4, 2, EPI, kDmaBK, kDmaStages, 8>;
      if (hipError_t e = DmaKernelLds<DT, 4, 2, EPI, kDmaBK, kDmaStages, 8>::entry.ensure(); e != hipSuccess) return e;
      hipLaunchKernelGGL(kern8, dim3(blocks), dim3(512), kDmaLds, s, g);
      return hipGetLastError();
    } else {
      auto kern = gemm_nt_dma_kernel<DT, TM, TN, EPI, kDmaBK, kDmaStages>;
      static_assert(kDmaLds == kDmaStages * (2 * TM * 32 + 2 * TN * 32) * kDmaBK * 2, "list entry and launch disagree");
      if (hipError_t e = DmaKernelLds<DT, TM, TN, EPI, kDmaBK, kDmaStages>::entry.ensure(); e != hipSuccess) return e;
      hipLaunchKernelGGL(kern, dim3(blocks), dim3(kGemmThreads), kDmaLds, s, g);
      return hipGetLastError();
    }
  }
  auto kern = gemm_nt_kernel<DT, TM, TN, EPI>;       // any K % 8 == 0: staged through registers
  if (hipError_t e = StagedKernelLds<DT, TM, TN, EPI>::entry.ensure(); e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(kGemmThreads), kLds, s, g);
  return hipGetLastError();
}

// Shape rule shared by the entry points: K a multiple of a 16-byte chunk (rows are fetched 16 bytes at a time).
static int check_gemm(int64_t M, int64_t N, int64_t K, int elem_bytes) {
  if (M < 0 || N <= 0 || K <= 0 || M > INT32_MAX / 2 || N > INT32_MAX / 2 || K > INT32_MAX / 2) return OMNI_ERR_SHAPE;
  if (K % (16 / elem_bytes) != 0) return OMNI_ERR_SHAPE;
  return OMNI_OK;
}

static int to_code(hipError_t e) { return e == hipSuccess ? OMNI_OK : OMNI_ERR_HIP_BASE + (int)e; }

// C[M,N] = A[M,K] B[N,K]^T (+ res), picking the tile shape from the problem size.
template <int DT>
static int gemm_plain(const void* a, const void* b, const void* b_hi, const void* res, void* c, int64_t M, int64_t N, int64_t K, hipStream_t s,
                      float* part_mean = nullptr, float* part_m2 = nullptr, bool exclusive = true) {
  if (int e = check_gemm(M, N, K, ElemBytes<DT>::value)) return e;
  if (M == 0) return OMNI_OK;
  GemmArgs g{(const uint8_t*)a, (const uint8_t*)b, (const uint8_t*)b_hi, (const uint8_t*)res, (uint8_t*)c, (int)M, (int)N, (int)K, 0, 0, 0, 0, 0, 0, nullptr, nullptr, nullptr};
  g.part_mean = part_mean;
  g.part_m2 = part_m2;
  g.exclusive = exclusive;
  const int64_t big = ((M + 255) / 256) * ((N + 255) / 256), mid = ((M + 127) / 128) * ((N + 127) / 128);
  hipError_t err;
  if (res) {
    if (big >= 200) err = launch_gemm<DT, 4, 4, kEpiResidual>(g, s);
    else if (mid >= 200) err = launch_gemm<DT, 2, 2, kEpiResidual>(g, s);
    else err = launch_gemm<DT, 1, 1, kEpiResidual>(g, s);
  } else if (part_mean) {
    if (big >= 200) err = launch_gemm<DT, 4, 4, kEpiStats>(g, s);
    else if (mid >= 200) err = launch_gemm<DT, 2, 2, kEpiStats>(g, s);
    else err = launch_gemm<DT, 1, 1, kEpiStats>(g, s);
  } else {
    if (big >= 200) err = launch_gemm<DT, 4, 4, kEpiPlain>(g, s);
    else if (mid >= 200) err = launch_gemm<DT, 2, 2, kEpiPlain>(g, s);
    else err = launch_gemm<DT, 1, 1, kEpiPlain>(g, s);
  }
  return to_code(err);
}

template <int DT>
static int gemm_swiglu(const void* x, const void* wg, const void* wu, void* h, int64_t M, int64_t I, int64_t K, hipStream_t s,
                       void* save_gate = nullptr, void* save_up = nullptr, bool exclusive = true) {
  if (int e = check_gemm(M, I, K, ElemBytes<DT>::value)) return e;
  if (M == 0) return OMNI_OK;
  GemmArgs g{(const uint8_t*)x, (const uint8_t*)wg, (const uint8_t*)wu, nullptr, (uint8_t*)h, (int)M, (int)I, (int)K, 0, 0, 0, 0, 0, 0, nullptr, nullptr, nullptr,
             (uint8_t*)save_gate, (uint8_t*)save_up};
  g.exclusive = exclusive;
  if (save_gate) {   // the saving epilogue has the 16-byte form only, in the direct-to-LDS kernel
    if (DT == kF32 || I % 8 != 0 || K % 64 != 0 || (uintptr_t)h % 16 || (uintptr_t)save_gate % 16 || (uintptr_t)save_up % 16) return OMNI_ERR_UNSUPPORTED;
  }
  const int64_t big = ((M + 255) / 256) * ((I + 127) / 128);
  hipError_t err;
  if (big >= 200) err = launch_gemm<DT, 4, 4, kEpiSwiglu>(g, s);
  else err = launch_gemm<DT, 2, 2, kEpiSwiglu>(g, s);
  return to_code(err);
}

}  // namespace omni

// c[T, 2N] = [round(v) | round(v - round(v))] with v = silu(x W^T) * gate, gate [T, N] fp32 (16-bit storage types only)
int omni_gemm_gated(const void* x, const void* w, const float* gate, void* c, int64_t T, int64_t N, int64_t K, int dtype, void* stream) {
  using namespace omni;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16) return OMNI_ERR_UNSUPPORTED;
  if (int e = check_gemm(T, N, K, 2)) return e;
  if (T == 0) return OMNI_OK;
  GemmArgs g{(const uint8_t*)x, (const uint8_t*)w, nullptr, nullptr, (uint8_t*)c, (int)T, (int)N, (int)K, 0, 0, 0, 0, 0, 0, nullptr, nullptr, gate};
  hipStream_t s = (hipStream_t)stream;
  const int64_t big = ((T + 255) / 256) * ((N + 255) / 256), mid = ((T + 127) / 128) * ((N + 127) / 128);
  hipError_t err;
  if (dtype == OMNI_BF16) {
    if (big >= 200) err = launch_gemm<kBF16, 4, 4, kEpiGate>(g, s);
    else if (mid >= 200) err = launch_gemm<kBF16, 2, 2, kEpiGate>(g, s);
    else err = launch_gemm<kBF16, 1, 1, kEpiGate>(g, s);
  } else {
    if (big >= 200) err = launch_gemm<kF16, 4, 4, kEpiGate>(g, s);
    else if (mid >= 200) err = launch_gemm<kF16, 2, 2, kEpiGate>(g, s);
    else err = launch_gemm<kF16, 1, 1, kEpiGate>(g, s);
  }
  return to_code(err);
}

int omni_gemm_router_projection(const void* x, const void* wx, const void* wy, void* z, float* part_mean, float* part_m2,
                                int64_t T, int H, int r, int dtype, void* stream) {
  using namespace omni;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == OMNI_BF16) return gemm_plain<kBF16>(x, wx, wy, nullptr, z, T, 2 * (int64_t)r, H, s, part_mean, part_m2);
  if (dtype == OMNI_F16) return gemm_plain<kF16>(x, wx, wy, nullptr, z, T, 2 * (int64_t)r, H, s, part_mean, part_m2);
  if (dtype == OMNI_F32) return gemm_plain<kF32>(x, wx, wy, nullptr, z, T, 2 * (int64_t)r, H, s, part_mean, part_m2);
  return OMNI_ERR_DTYPE;
}

extern "C" OMNI_API size_t omni_mlp_workspace_bytes(int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size, int32_t dtype) {
  (void)hidden_size;
  if (num_tokens < 0 || intermediate_size < 0) return 0;
  const size_t es = dtype == OMNI_F32 ? 4 : 2;
  return (size_t)num_tokens * (size_t)intermediate_size * es;      // h = silu(gate)*up
}

extern "C" OMNI_API int32_t omni_mlp_fwd(const void* x, const void* gate_weight, const void* up_weight, const void* down_weight,
                                         const void* residual, void* y, int64_t num_tokens, int32_t hidden_size,
                                         int32_t intermediate_size, int32_t dtype, void* workspace, void* stream) {
  using namespace omni;
  if (num_tokens < 0 || hidden_size <= 0 || intermediate_size <= 0) return OMNI_ERR_SHAPE;
  if (num_tokens == 0) return OMNI_OK;
  if (!x || !gate_weight || !up_weight || !down_weight || !y) return OMNI_ERR_NULL;
  if (!workspace) return OMNI_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  int e;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  // both projections are checked before the first one is enqueued: hidden and intermediate size are each the K of one
  const int es = dtype == OMNI_F32 ? 4 : 2;
  if ((e = check_gemm(num_tokens, intermediate_size, hidden_size, es)) || (e = check_gemm(num_tokens, hidden_size, intermediate_size, es)))
    return e;
  switch (dtype) {
    case OMNI_BF16:
      if ((e = gemm_swiglu<kBF16>(x, gate_weight, up_weight, workspace, num_tokens, intermediate_size, hidden_size, s))) return e;
      return gemm_plain<kBF16>(workspace, down_weight, nullptr, residual, y, num_tokens, hidden_size, intermediate_size, s);
    case OMNI_F16:
      if ((e = gemm_swiglu<kF16>(x, gate_weight, up_weight, workspace, num_tokens, intermediate_size, hidden_size, s))) return e;
      return gemm_plain<kF16>(workspace, down_weight, nullptr, residual, y, num_tokens, hidden_size, intermediate_size, s);
    case OMNI_F32:
      if ((e = gemm_swiglu<kF32>(x, gate_weight, up_weight, workspace, num_tokens, intermediate_size, hidden_size, s))) return e;
      return gemm_plain<kF32>(workspace, down_weight, nullptr, residual, y, num_tokens, hidden_size, intermediate_size, s);
    default: return OMNI_ERR_DTYPE;
  }
}

// The two projection calls with the caller's word on whether anything runs beside them (the whole-layer call on two
// streams says no to `exclusive`, which keeps the GEMMs off the streaming form that would hold every CU).
namespace omni {
int swiglu_linear_fwd_impl(const void* x, const void* gate_weight, const void* up_weight, void* h, int64_t num_tokens,
                           int32_t hidden_size, int32_t intermediate_size, int32_t dtype, void* stream, bool exclusive) {
  if (num_tokens == 0) return OMNI_OK;
  if (!x || !gate_weight || !up_weight || !h) return OMNI_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case OMNI_BF16: return gemm_swiglu<kBF16>(x, gate_weight, up_weight, h, num_tokens, intermediate_size, hidden_size, s, nullptr, nullptr, exclusive);
    case OMNI_F16: return gemm_swiglu<kF16>(x, gate_weight, up_weight, h, num_tokens, intermediate_size, hidden_size, s, nullptr, nullptr, exclusive);
    case OMNI_F32: return gemm_swiglu<kF32>(x, gate_weight, up_weight, h, num_tokens, intermediate_size, hidden_size, s, nullptr, nullptr, exclusive);
    default: return OMNI_ERR_DTYPE;
  }
}
int linear_fwd_impl(const void* x, const void* weight, const void* residual, void* y, int64_t num_tokens, int32_t in_features,
                    int32_t out_features, int32_t dtype, void* stream, bool exclusive) {
  if (num_tokens == 0) return OMNI_OK;
  if (!x || !weight || !y) return OMNI_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case OMNI_BF16: return gemm_plain<kBF16>(x, weight, nullptr, residual, y, num_tokens, out_features, in_features, s, nullptr, nullptr, exclusive);
    case OMNI_F16: return gemm_plain<kF16>(x, weight, nullptr, residual, y, num_tokens, out_features, in_features, s, nullptr, nullptr, exclusive);
    case OMNI_F32: return gemm_plain<kF32>(x, weight, nullptr, residual, y, num_tokens, out_features, in_features, s, nullptr, nullptr, exclusive);
    default: return OMNI_ERR_DTYPE;
  }
}
}  // namespace omni

extern "C" OMNI_API int32_t omni_swiglu_linear_fwd(const void* x, const void* gate_weight, const void* up_weight, void* h,
                                                   int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size,
                                                   int32_t dtype, void* stream) {
  return omni::swiglu_linear_fwd_impl(x, gate_weight, up_weight, h, num_tokens, hidden_size, intermediate_size, dtype, stream, true);
}

extern "C" OMNI_API int32_t omni_swiglu_linear_fwd_shared(const void* x, const void* gate_weight, const void* up_weight, void* h,
                                                          int64_t num_tokens, int32_t hidden_size, int32_t intermediate_size,
                                                          int32_t dtype, void* stream) {
  return omni::swiglu_linear_fwd_impl(x, gate_weight, up_weight, h, num_tokens, hidden_size, intermediate_size, dtype, stream, false);
}

extern "C" OMNI_API int32_t omni_swiglu_linear_save_fwd(const void* x, const void* gate_weight, const void* up_weight, void* h,
                                                        void* gate_out, void* up_out, int64_t num_tokens, int32_t hidden_size,
                                                        int32_t intermediate_size, int32_t dtype, void* stream) {
  using namespace omni;
  if (num_tokens == 0) return OMNI_OK;
  if (!x || !gate_weight || !up_weight || !h || !gate_out || !up_out) return OMNI_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case OMNI_BF16: return gemm_swiglu<kBF16>(x, gate_weight, up_weight, h, num_tokens, intermediate_size, hidden_size, s, gate_out, up_out);
    case OMNI_F16: return gemm_swiglu<kF16>(x, gate_weight, up_weight, h, num_tokens, intermediate_size, hidden_size, s, gate_out, up_out);
    case OMNI_F32: return OMNI_ERR_UNSUPPORTED;
    default: return OMNI_ERR_DTYPE;
  }
}

extern "C" OMNI_API int32_t omni_linear_fwd(const void* x, const void* weight, const void* residual, void* y, int64_t num_tokens,
                                            int32_t in_features, int32_t out_features, int32_t dtype, void* stream) {
  return omni::linear_fwd_impl(x, weight, residual, y, num_tokens, in_features, out_features, dtype, stream, true);
}

extern "C" OMNI_API int32_t omni_linear2_fwd(const void* x, const void* weight_lo, const void* weight_hi, void* y,
                                             int64_t num_tokens, int32_t in_features, int32_t out_features_each,
                                             int32_t dtype, void* stream) {
  using namespace omni;
  if (num_tokens == 0) return OMNI_OK;
  if (!x || !weight_lo || !weight_hi || !y) return OMNI_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  const int64_t n = 2 * (int64_t)out_features_each;
  switch (dtype) {
    case OMNI_BF16: return gemm_plain<kBF16>(x, weight_lo, weight_hi, nullptr, y, num_tokens, n, in_features, s);
    case OMNI_F16: return gemm_plain<kF16>(x, weight_lo, weight_hi, nullptr, y, num_tokens, n, in_features, s);
    case OMNI_F32: return gemm_plain<kF32>(x, weight_lo, weight_hi, nullptr, y, num_tokens, n, in_features, s);
    default: return OMNI_ERR_DTYPE;
  }
}

namespace omni {
// y[i] = round(y[i] + e[i]), 8 (16-bit) or 4 (fp32) elements per lane
template <int DT>
__global__ __launch_bounds__(256) void add_inplace_kernel(uint8_t* __restrict__ y, const uint8_t* __restrict__ e, int64_t num_chunks) {
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < num_chunks; i += gridDim.x * 256ll) {
    const u32x4_t a = *(const u32x4_t*)(y + i * 16), b = *(const u32x4_t*)(e + i * 16);
    u32x4_t o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t aq = a[q], bq = b[q];
      if constexpr (DT == kBF16) o[q] = pack_bf16(bf16_lo(aq) + bf16_lo(bq), bf16_hi(aq) + bf16_hi(bq));
      else if constexpr (DT == kF16) o[q] = pack_f16(f16_bits_to_f32(aq & 0xffff) + f16_bits_to_f32(bq & 0xffff), f16_bits_to_f32(aq >> 16) + f16_bits_to_f32(bq >> 16));
      else o[q] = __float_as_uint(__uint_as_float(aq) + __uint_as_float(bq));
    }
    *(u32x4_t*)(y + i * 16) = o;
  }
}
}  // namespace omni

extern "C" OMNI_API int32_t omni_add_inplace(void* y, const void* addend, int64_t num_elements, int32_t dtype, void* stream) {
  using namespace omni;
  if (num_elements < 0) return OMNI_ERR_SHAPE;
  if (dtype != OMNI_BF16 && dtype != OMNI_F16 && dtype != OMNI_F32) return OMNI_ERR_DTYPE;
  const int per = dtype == OMNI_F32 ? 4 : 8;
  if (num_elements % per != 0) return OMNI_ERR_SHAPE;
  if (num_elements == 0) return OMNI_OK;
  if (!y || !addend) return OMNI_ERR_NULL;
  const int64_t chunks = num_elements / per;
  const unsigned blocks = (unsigned)((chunks + 255) / 256 < 4096 ? (chunks + 255) / 256 : 4096);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == OMNI_BF16) hipLaunchKernelGGL(add_inplace_kernel<kBF16>, dim3(blocks), dim3(256), 0, s, (uint8_t*)y, (const uint8_t*)addend, chunks);
  else if (dtype == OMNI_F16) hipLaunchKernelGGL(add_inplace_kernel<kF16>, dim3(blocks), dim3(256), 0, s, (uint8_t*)y, (const uint8_t*)addend, chunks);
  else hipLaunchKernelGGL(add_inplace_kernel<kF32>, dim3(blocks), dim3(256), 0, s, (uint8_t*)y, (const uint8_t*)addend, chunks);
  return omni::to_code(hipGetLastError());
}

namespace omni {
// Matrix-core rate with nothing else going on: every wave keeps 16 accumulator tiles and issues
// MFMAs on operands it read once (8 KiB of caller data, so that the operand bits are realistic:
// the sustained clock under the board's power limit depends on how many bits toggle).
__global__ __launch_bounds__(kGemmThreads, 1) void mfma_probe_kernel(const u32x4_t* __restrict__ operands, float* __restrict__ sink, int iters) {
  f32x16_t acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int q = 0; q < 16; ++q) acc[i][q] = 0.f;
  u32x4_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operands[(threadIdx.x * 8 + i) & 511];
    b[i] = operands[(threadIdx.x * 8 + 4 + i) & 511];
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = mfma32<kBF16>(a[i & 3], b[i >> 2], acc[i]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i][0] + acc[i][5];
  sink[blockIdx.x * kGemmThreads + threadIdx.x] = s;
}
// The same with v_mfma_f32_16x16x32_bf16, the streaming kernel's instruction: 8 waves per block (two per SIMD, as that
// kernel runs), 8 x 4 independent accumulator tiles per wave.
__global__ __launch_bounds__(512, 1) void mfma_probe16_kernel(const u32x4_t* __restrict__ operands, float* __restrict__ sink, int iters) {
  f32x4_t acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) acc[i][j][q] = 0.f;
  u32x4_t a[8], b[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = operands[(threadIdx.x * 12 + i) & 511];
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = operands[(threadIdx.x * 12 + 8 + i) & 511];
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = mfma16<kBF16>(b[j], a[i], acc[i][j]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) s += acc[i][j][0] + acc[i][j][3];
  sink[blockIdx.x * 512 + threadIdx.x] = s;
}
}  // namespace omni

extern "C" OMNI_API int32_t omni_probe_mfma16(const void* operands, float* sink, int32_t num_blocks, int32_t iters, void* stream) {
  if (num_blocks <= 0 || iters <= 0) return OMNI_ERR_SHAPE;
  if (!operands || !sink) return OMNI_ERR_NULL;
  hipLaunchKernelGGL(omni::mfma_probe16_kernel, dim3(num_blocks), dim3(512), 0, (hipStream_t)stream, (const omni::u32x4_t*)operands, sink, iters);
  return omni::to_code(hipGetLastError());
}

extern "C" OMNI_API int32_t omni_probe_mfma(const void* operands, float* sink, int32_t num_blocks, int32_t iters, void* stream) {
  if (num_blocks <= 0 || iters <= 0) return OMNI_ERR_SHAPE;
  if (!operands || !sink) return OMNI_ERR_NULL;
  hipLaunchKernelGGL(omni::mfma_probe_kernel, dim3(num_blocks), dim3(omni::kGemmThreads), 0, (hipStream_t)stream,
                     (const omni::u32x4_t*)operands, sink, iters);
  return omni::to_code(hipGetLastError());
}

