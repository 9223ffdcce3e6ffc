// Paged KV-cache write kernels (gfx950).
//
// pa_kv_store      same-dtype scatter copy of token rows into cache slots
//                  (reference: src/inference/attention.py:119-135 and 141-183)
// pa_kv_store_fp8  per-token amax -> scale = (1/amax)*448 -> e4m3fn bytes + fp32 scale
//                  (reference: src/inference/attention.py:75-116)
//
// Both are latency-bound (a decode step moves 128 KiB per tensor at batch 64), so the
// kernels aim at one short launch: K and V in the same grid, 16-byte accesses, one
// wavefront per (token, tensor) row for the quantising writer so the amax reduction
// never leaves the wave.
#include "pa_common.hpp"
#include "pa_host.hpp"

namespace pa {

// ---- bit copy ------------------------------------------------------------------------

// grid.x = token, grid.y = 0 (K) / 1 (V); the row is moved in 16-byte pieces.
__global__ __launch_bounds__(128) void kv_store_copy_kernel(
    const uint8_t* __restrict__ key, const uint8_t* __restrict__ value, int64_t key_stride_b,
    int64_t value_stride_b, uint8_t* __restrict__ k_cache, uint8_t* __restrict__ v_cache,
    const int32_t* __restrict__ slot_mapping, int64_t row_bytes, int64_t total_slots) {
  const int64_t t = blockIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0 || slot >= total_slots) return;
  const bool is_v = blockIdx.y != 0;
  const uint8_t* src = is_v ? value + t * value_stride_b : key + t * key_stride_b;
  uint8_t* dst = (is_v ? v_cache : k_cache) + slot * row_bytes;
  for (int64_t off = (int64_t)threadIdx.x * 16; off < row_bytes; off += 128 * 16) {
    *(uint4*)(dst + off) = *(const uint4*)(src + off);
  }
}

// ---- fp8 quantising write --------------------------------------------------------------

// max that keeps NaN once seen (torch.amax propagates NaN).
__device__ __forceinline__ float nan_max(float m, float a) { return (a > m || a != a) ? a : m; }

template <int IN_DTYPE>
__device__ __forceinline__ void load16(const void* row, int64_t e0, float (&x)[16]) {
  if constexpr (IN_DTYPE == PA_DTYPE_F32) {
    const float4* p = (const float4*)((const float*)row + e0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float4 v = p[i];
      x[4 * i + 0] = v.x;
      x[4 * i + 1] = v.y;
      x[4 * i + 2] = v.z;
      x[4 * i + 3] = v.w;
    }
  } else {
    const uint4* p = (const uint4*)((const uint16_t*)row + e0);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      uint4 v = p[i];
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if constexpr (IN_DTYPE == PA_DTYPE_F16) {
          x[8 * i + 2 * k + 0] = f16_bits_to_f32(w[k] & 0xffffu);
          x[8 * i + 2 * k + 1] = f16_bits_to_f32(w[k] >> 16);
        } else {
          x[8 * i + 2 * k + 0] = bf16_bits_to_f32(w[k] & 0xffffu);
          x[8 * i + 2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
        }
      }
    }
  }
}

// One wavefront per (token, K|V) row: lane l owns elements [16*(l + 64*c), +16) for c = 0,1,..
// so every lane stores 16 contiguous bytes.  The first chunk stays in registers between the
// amax pass and the encode pass; longer rows re-read the rest (L2 hits).
template <int IN_DTYPE>
__global__ __launch_bounds__(256) void kv_store_fp8_kernel(
    const void* __restrict__ key, const void* __restrict__ value, int64_t key_stride,
    int64_t value_stride, uint8_t* __restrict__ k_cache, uint8_t* __restrict__ v_cache,
    float* __restrict__ k_scale, float* __restrict__ v_scale,
    const int32_t* __restrict__ slot_mapping, int64_t num_tokens, int64_t row_elems,
    int64_t total_slots) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t row_id = (int64_t)blockIdx.x * 4 + wave;  // 2 rows (K,V) per token
  const int64_t t = row_id >> 1;
  if (t >= num_tokens) return;
  const bool is_v = (row_id & 1) != 0;
  const int64_t slot = slot_mapping[t];
  if (slot < 0 || slot >= total_slots) return;

  constexpr int ES = IN_DTYPE == PA_DTYPE_F32 ? 4 : 2;
  const uint8_t* src =
      (const uint8_t*)(is_v ? value : key) + t * (is_v ? value_stride : key_stride) * ES;
  uint8_t* dst = (is_v ? v_cache : k_cache) + slot * row_elems;
  float* scale_dst = (is_v ? v_scale : k_scale) + slot;

  float x0[16];
  float amax = 0.0f;
  const int64_t e_first = (int64_t)lane * 16;
  const bool has_first = e_first < row_elems;
  if (has_first) {
    load16<IN_DTYPE>(src, e_first, x0);
#pragma unroll
    for (int i = 0; i < 16; ++i) amax = nan_max(amax, fabsf(x0[i]));
  }
  for (int64_t e = e_first + 1024; e < row_elems; e += 1024) {
    float x[16];
    load16<IN_DTYPE>(src, e, x);
#pragma unroll
    for (int i = 0; i < 16; ++i) amax = nan_max(amax, fabsf(x[i]));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = nan_max(amax, __shfl_xor(amax, o));

  amax = amax < 1e-5f ? 1e-5f : amax;        // clamp(min=1e-5); NaN stays NaN
  // torch evaluates `448.0 / amax` (python scalar over a tensor) as amax.reciprocal() * 448.0:
  // a correctly rounded fp32 reciprocal followed by a separately rounded fp32 multiply.
  const float s = __fmul_rn(__fdiv_rn(1.0f, amax), 448.0f);
  if (lane == 0) *scale_dst = s;

  // The scaled values never exceed 448 by more than a rounding (the largest element times 448 / amax),
  // and on that range - and for NaN - the hardware conversion (v_cvt_pk_fp8_f32: OCP e4m3fn on gfx950,
  // round to nearest even, subnormals, signed zero) gives the bytes of the reference's cast; what it does
  // beyond 464, where the reference's cast makes NaN, cannot be reached from here.
  auto encode_store = [&](const float(&x)[16], int64_t e) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int b = 0;
      b = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(x[4 * i], s), __fmul_rn(x[4 * i + 1], s), b, false);
      b = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(x[4 * i + 2], s), __fmul_rn(x[4 * i + 3], s), b, true);
      w[i] = (uint32_t)b;
    }
    *(uint4*)(dst + e) = make_uint4(w[0], w[1], w[2], w[3]);
  };
  if (has_first) encode_store(x0, e_first);
  for (int64_t e = e_first + 1024; e < row_elems; e += 1024) {
    float x[16];
    load16<IN_DTYPE>(src, e, x);
    encode_store(x, e);
  }
}

// ---- element-wise converters (exposed for checking cache contents) ----------------------

__global__ void fp8_to_f32_kernel(const uint8_t* __restrict__ src, float* __restrict__ dst,
                                  int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t b = src[i];
  dst[i] = fp8x2_to_f32(b, false)[0];
}

__global__ void f32_to_fp8_kernel(const float* __restrict__ src, uint8_t* __restrict__ dst,
                                  int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  dst[i] = (uint8_t)f32_to_e4m3fn(src[i]);
}

}  // namespace pa

using namespace pa;

extern "C" int pa_kv_store(const void* key, const void* value, int64_t key_token_stride,
                           int64_t value_token_stride, void* k_cache, void* v_cache,
                           const int32_t* slot_mapping, int64_t num_tokens, int64_t row_elems,
                           int elem_bytes, int64_t total_slots, void* stream) {
  if (num_tokens < 0 || row_elems <= 0 || total_slots < 0)
    return fail(PA_ERR_BAD_ARG, "pa_kv_store: negative size");
  if (num_tokens == 0) return PA_OK;
  if (!key || !value || !k_cache || !v_cache || !slot_mapping)
    return fail(PA_ERR_BAD_ARG, "pa_kv_store: null pointer");
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4)
    return fail(PA_ERR_UNSUPPORTED, "pa_kv_store: elem_bytes must be 1, 2 or 4");
  const int64_t row_bytes = row_elems * elem_bytes;
  if (row_bytes % 16 != 0 || (key_token_stride * elem_bytes) % 16 != 0 ||
      (value_token_stride * elem_bytes) % 16 != 0)
    return fail(PA_ERR_UNSUPPORTED, "pa_kv_store: rows and token strides must be multiples of 16 bytes");
  if (!aligned16(key) || !aligned16(value) || !aligned16(k_cache) || !aligned16(v_cache))
    return fail(PA_ERR_BAD_ARG, "pa_kv_store: buffers must be 16-byte aligned");
  if (key_token_stride < row_elems || value_token_stride < row_elems)
    return fail(PA_ERR_BAD_ARG, "pa_kv_store: token stride smaller than the row");
  if (num_tokens > 0x7fffffff) return fail(PA_ERR_UNSUPPORTED, "pa_kv_store: too many tokens");
  dim3 grid((unsigned)num_tokens, 2);
  hipLaunchKernelGGL(kv_store_copy_kernel, grid, dim3(128), 0, (hipStream_t)stream,
                     (const uint8_t*)key, (const uint8_t*)value, key_token_stride * elem_bytes,
                     value_token_stride * elem_bytes, (uint8_t*)k_cache, (uint8_t*)v_cache,
                     slot_mapping, row_bytes, total_slots);
  return check_launch("pa_kv_store");
}

extern "C" int pa_kv_store_fp8(const void* key, const void* value, int in_dtype,
                               int64_t key_token_stride, int64_t value_token_stride,
                               void* k_cache, void* v_cache, float* k_scale, float* v_scale,
                               const int32_t* slot_mapping, int64_t num_tokens,
                               int64_t row_elems, int64_t total_slots, void* stream) {
  if (num_tokens < 0 || row_elems <= 0 || total_slots < 0)
    return fail(PA_ERR_BAD_ARG, "pa_kv_store_fp8: negative size");
  if (num_tokens == 0) return PA_OK;
  if (!key || !value || !k_cache || !v_cache || !k_scale || !v_scale || !slot_mapping)
    return fail(PA_ERR_BAD_ARG, "pa_kv_store_fp8: null pointer (fp8 needs k_scale and v_scale)");
  if (row_elems % 16 != 0 || key_token_stride % 16 != 0 || value_token_stride % 16 != 0)
    return fail(PA_ERR_UNSUPPORTED, "pa_kv_store_fp8: row_elems and token strides must be multiples of 16");
  if (!aligned16(key) || !aligned16(value) || !aligned16(k_cache) || !aligned16(v_cache))
    return fail(PA_ERR_BAD_ARG, "pa_kv_store_fp8: buffers must be 16-byte aligned");
  if (key_token_stride < row_elems || value_token_stride < row_elems)
    return fail(PA_ERR_BAD_ARG, "pa_kv_store_fp8: token stride smaller than the row");
  const int64_t rows = num_tokens * 2;
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffff) return fail(PA_ERR_UNSUPPORTED, "pa_kv_store_fp8: too many tokens");
  dim3 grid((unsigned)blocks), block(256);
  hipStream_t st = (hipStream_t)stream;
#define PA_LAUNCH_FP8(DT)                                                                      \
  hipLaunchKernelGGL(kv_store_fp8_kernel<DT>, grid, block, 0, st, key, value, key_token_stride, \
                     value_token_stride, (uint8_t*)k_cache, (uint8_t*)v_cache, k_scale, v_scale, \
                     slot_mapping, num_tokens, row_elems, total_slots)
  switch (in_dtype) {
    case PA_DTYPE_F16: PA_LAUNCH_FP8(PA_DTYPE_F16); break;
    case PA_DTYPE_BF16: PA_LAUNCH_FP8(PA_DTYPE_BF16); break;
    case PA_DTYPE_F32: PA_LAUNCH_FP8(PA_DTYPE_F32); break;
    default: return fail(PA_ERR_UNSUPPORTED, "pa_kv_store_fp8: in_dtype must be f16, bf16 or f32");
  }
#undef PA_LAUNCH_FP8
  return check_launch("pa_kv_store_fp8");
}

extern "C" int pa_fp8_e4m3_to_f32(const void* src, float* dst, int64_t n, void* stream) {
  if (n < 0) return fail(PA_ERR_BAD_ARG, "pa_fp8_e4m3_to_f32: negative size");
  if (n == 0) return PA_OK;
  if (!src || !dst) return fail(PA_ERR_BAD_ARG, "pa_fp8_e4m3_to_f32: null pointer");
  const int64_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffff) return fail(PA_ERR_UNSUPPORTED, "pa_fp8_e4m3_to_f32: too large");
  hipLaunchKernelGGL(fp8_to_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)src, dst, n);
  return check_launch("pa_fp8_e4m3_to_f32");
}

extern "C" int pa_f32_to_fp8_e4m3(const float* src, void* dst, int64_t n, void* stream) {
  if (n < 0) return fail(PA_ERR_BAD_ARG, "pa_f32_to_fp8_e4m3: negative size");
  if (n == 0) return PA_OK;
  if (!src || !dst) return fail(PA_ERR_BAD_ARG, "pa_f32_to_fp8_e4m3: null pointer");
  const int64_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffff) return fail(PA_ERR_UNSUPPORTED, "pa_f32_to_fp8_e4m3: too large");
  hipLaunchKernelGGL(f32_to_fp8_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     src, (uint8_t*)dst, n);
  return check_launch("pa_f32_to_fp8_e4m3");
}
