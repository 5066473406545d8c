// Row arithmetic shared by the expert kernels: a wave walks a row of H elements 16 bytes per
// lane per KiB; these helpers work on one such 16-byte piece (8 x 16-bit or 4 x fp32).
#pragma once
#include "common.h"

namespace omni {

template <int DT> struct Row16 {               // what one 16-byte lane load holds
  static constexpr int kElems = (DT == kF32) ? 4 : 8;
};

template <int DT>
__device__ __forceinline__ float dot16(const u32x4_t a, const u32x4_t b, float acc) {
  if constexpr (DT == kBF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t ai = a[i], bi = b[i];     // bit_cast wants a scalar object, not a vector element
      acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, ai), __builtin_bit_cast(bf16x2_t, bi), acc, false);
    }
  } else if constexpr (DT == kF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t ai = a[i], bi = b[i];
      acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, ai), __builtin_bit_cast(f16x2_t, bi), acc, false);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = fmaf(__uint_as_float(a[i]), __uint_as_float(b[i]), acc);
  }
  return acc;
}

// acc[0..kElems) += c * row
template <int DT>
__device__ __forceinline__ void axpy16(float c, const u32x4_t v, float* acc) {
  if constexpr (DT == kBF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t vi = v[i];
      acc[2 * i] = fmaf(c, bf16_lo(vi), acc[2 * i]);
      acc[2 * i + 1] = fmaf(c, bf16_hi(vi), acc[2 * i + 1]);
    }
  } else if constexpr (DT == kF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t vi = v[i];
      f16x2_t p = __builtin_bit_cast(f16x2_t, vi);
      acc[2 * i] = fmaf(c, float(p[0]), acc[2 * i]);
      acc[2 * i + 1] = fmaf(c, float(p[1]), acc[2 * i + 1]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = fmaf(c, __uint_as_float(v[i]), acc[i]);
  }
}

template <int DT>
__device__ __forceinline__ u32x4_t pack16(const float* acc) {
  u32x4_t o;
  if constexpr (DT == kBF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack_bf16(acc[2 * i], acc[2 * i + 1]);
  } else if constexpr (DT == kF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack_f16(acc[2 * i], acc[2 * i + 1]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = __float_as_uint(acc[i]);
  }
  return o;
}

// the elements of a 16-byte piece as floats
template <int DT>
__device__ __forceinline__ void unpack16(const u32x4_t v, float* out) {
  if constexpr (DT == kBF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t vi = v[i];
      out[2 * i] = bf16_lo(vi);
      out[2 * i + 1] = bf16_hi(vi);
    }
  } else if constexpr (DT == kF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t vi = v[i];
      const f16x2_t p = __builtin_bit_cast(f16x2_t, vi);
      out[2 * i] = float(p[0]);
      out[2 * i + 1] = float(p[1]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = __uint_as_float(v[i]);
  }
}

}  // namespace omni
