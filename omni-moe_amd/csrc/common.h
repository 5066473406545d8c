// Device-side helpers shared by the gfx950 kernels of the OmniMoE forward path.
// Wave size is 64 throughout; nothing here is written for any other target.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace omni {

constexpr int kWave = 64;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// Storage dtypes of the operator API (values match include/omni_moe_hip.h).
enum : int { kBF16 = 0, kF16 = 1, kF32 = 2 };

// ---- scalar conversions ----------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(uint32_t(b) << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t p) { return __uint_as_float(p << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t p) { return __uint_as_float(p & 0xffff0000u); }

// two floats -> packed bf16 pair, round-to-nearest-even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  f32x2_t f = {lo, hi};
  bf16x2_t r = __builtin_convertvector(f, bf16x2_t);
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return uint16_t(pack_bf16(f, 0.f) & 0xffffu); }
__device__ __forceinline__ float round_to_bf16(float f) { return bf16_lo(pack_bf16(f, 0.f)); }

__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) { return float(__builtin_bit_cast(_Float16, b)); }
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __builtin_bit_cast(uint16_t, _Float16(f)); }
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  return uint32_t(f32_to_f16_bits(lo)) | (uint32_t(f32_to_f16_bits(hi)) << 16);
}

// Per-dtype element traits used by the bandwidth-bound kernels.
template <int DT> struct Elem;
template <> struct Elem<kBF16> {
  typedef uint16_t store_t;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return bf16_bits_to_f32(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = f32_to_bf16_bits(v); }
  static __device__ __forceinline__ float round(float v) { return round_to_bf16(v); }
};
template <> struct Elem<kF16> {
  typedef uint16_t store_t;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return f16_bits_to_f32(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = f32_to_f16_bits(v); }
  static __device__ __forceinline__ float round(float v) { return float(_Float16(v)); }
};
template <> struct Elem<kF32> {
  typedef float store_t;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};

// ---- wave-level primitives ---------------------------------------------------
__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, kWave));
  return v;
}

// Value of lane (lane ^ STRIDE) without touching LDS memory: DPP quad permutes (1, 2), two
// bank-masked DPP row shifts (4, 8), a ds_swizzle bit pattern (16), v_permlane32_swap (32).
template <int STRIDE>
__device__ __forceinline__ int xor_lane_i(int v, int lane) {
  if constexpr (STRIDE == 1) return __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xf, 0xf, false);
  else if constexpr (STRIDE == 2) return __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xf, 0xf, false);
  else if constexpr (STRIDE == 4) {
    const int t = __builtin_amdgcn_update_dpp(v, v, 0x104, 0xf, 0x5, false);     // row_shl:4 into banks 0,2
    return __builtin_amdgcn_update_dpp(t, v, 0x114, 0xf, 0xA, false);            // row_shr:4 into banks 1,3
  } else if constexpr (STRIDE == 8) {
    const int t = __builtin_amdgcn_update_dpp(v, v, 0x108, 0xf, 0x3, false);     // row_shl:8 into banks 0,1
    return __builtin_amdgcn_update_dpp(t, v, 0x118, 0xf, 0xC, false);            // row_shr:8 into banks 2,3
  } else if constexpr (STRIDE == 16) return __builtin_amdgcn_ds_swizzle(v, 0x401F);
  else {
    const auto sw = __builtin_amdgcn_permlane32_swap(v, v, false, false);         // [lo,lo] and [hi,hi]
    return (lane & 32) ? (int)sw[0] : (int)sw[1];
  }
}
template <int STRIDE>
__device__ __forceinline__ float xor_lane_f(float v, int lane) {
  return __int_as_float(xor_lane_i<STRIDE>(__float_as_int(v), lane));
}

// x*sigmoid(x) in fp32, IEEE division.
__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + __expf(-x)); }
// Same with the hardware reciprocal (1 ulp) and exp2: ~6 instructions.  For results that are
// rounded to a 16-bit type straight away.
__device__ __forceinline__ float silu_fast(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// ---- host side ---------------------------------------------------------------
// A kernel whose dynamic LDS exceeds the 64 KiB default needs its limit raised once per device (the
// attribute belongs to the device's copy of the kernel).  Every such kernel is one LdsKernel object with
// static storage: its constructor links it into a list at library load, so that omni_init() can raise all
// limits up front (a caller that captures HIP graphs wants no hipFuncSetAttribute inside a capture), and
// ensure() does it on first use for callers that never call omni_init().  `done` is the bit mask of devices
// already set up; concurrent callers at worst set the attribute twice.
struct LdsKernel;
inline LdsKernel*& lds_kernel_list() {
  static LdsKernel* head = nullptr;
  return head;
}
struct LdsKernel {
  const void* kernel;
  int bytes;
  std::atomic<uint64_t> done{0};
  LdsKernel* next;
  LdsKernel(const void* k, int b) : kernel(k), bytes(b), next(lds_kernel_list()) { lds_kernel_list() = this; }
  hipError_t ensure() {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    if (hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes); e != hipSuccess) return e;
    done.fetch_or(bit, std::memory_order_release);
    return hipSuccess;
  }
};

// The schedule's allocation-free entry point keeps a device array; this resolves its address on the
// current device (defined beside the array).
int schedule_scratch_prepare();

}  // namespace omni
