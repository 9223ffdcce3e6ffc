// Shared device helpers for the gfx950 paged-attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "paged_attn.h"

namespace pa {

constexpr int kWave = 64;

enum : int { KV_F16 = 0, KV_BF16 = 1, KV_FP8 = 2 };

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

// ---- scalar conversions -------------------------------------------------------------

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// fp32 -> bf16 bits, round-to-nearest-even (NaN kept quiet).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// Read element i of a tensor of type `dtype` (PA_DTYPE_F16/BF16/F32) as fp32.
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i, int dtype) {
  if (dtype == PA_DTYPE_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
  if (dtype == PA_DTYPE_BF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

// Eight consecutive elements starting at index i (i % 8 == 0, base 16-byte aligned) as fp32.
__device__ __forceinline__ void load8_as_f32(const void* p, int64_t i, int dtype, float (&x)[8]) {
  if (dtype == PA_DTYPE_F32) {
    const float4 a = *(const float4*)((const float*)p + i);
    const float4 b = *(const float4*)((const float*)p + i + 4);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
  } else {
    const uint4 v = *(const uint4*)((const uint16_t*)p + i);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (dtype == PA_DTYPE_F16) {
        x[2 * k] = f16_bits_to_f32(w[k] & 0xffffu);
        x[2 * k + 1] = f16_bits_to_f32(w[k] >> 16);
      } else {
        x[2 * k] = bf16_bits_to_f32(w[k] & 0xffffu);
        x[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
      }
    }
  }
}

__device__ __forceinline__ void store_from_f32(void* p, int64_t i, int dtype, float v) {
  if (dtype == PA_DTYPE_F16)
    ((uint16_t*)p)[i] = f32_to_f16_bits(v);
  else if (dtype == PA_DTYPE_BF16)
    ((uint16_t*)p)[i] = f32_to_bf16_bits(v);
  else
    ((float*)p)[i] = v;
}

// ---- fp8 e4m3fn ---------------------------------------------------------------------

// Two e4m3fn bytes (low or high half of a dword) -> two fp32; exact.
__device__ __forceinline__ float2_t fp8x2_to_f32(uint32_t w, bool hi) {
  return hi ? __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true)
            : __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
}

// fp32 -> e4m3fn byte: round-to-nearest-even on the 3-bit mantissa, subnormals down to
// 2^-9, no saturation (|x| that rounds beyond 448, infinities and NaN give 0x7F | sign).
__device__ __forceinline__ uint32_t f32_to_e4m3fn(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t sign = (u >> 24) & 0x80u;
  const uint32_t a = u & 0x7fffffffu;
  uint32_t r;
  if (a >= 0x43f00000u) {  // |x| >= 480 (first value that cannot round to 448), inf, NaN
    r = 0x7fu;
  } else if (a < 0x3c800000u) {  // |x| < 2^-6: subnormal grid of 2^-9, RNE to an integer step
    r = (uint32_t)__float2int_rn(__uint_as_float(a) * 512.0f);
  } else {
    // keep 3 mantissa bits: add half an output ulp minus one, plus the parity of the kept lsb
    const uint32_t rounded = a + 0x7ffffu + ((a >> 20) & 1u);
    r = (rounded >> 20) - ((127u - 7u) << 3);
  }
  return r | sign;
}

// ---- cross-lane ---------------------------------------------------------------------

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// Sum over each aligned group of 8 lanes; every lane of the group gets the total.
__device__ __forceinline__ float sum8(float v) {
  v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f32<0x141>(v);  // row_half_mirror: lane i <-> 7-i inside each half row
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}

}  // namespace pa
