// Per-head q/k RMSNorm + rotary embedding + paged KV-cache write in one launch (gfx950).
//
// What a Qwen3 attention block does between its q/k/v projections and the attention call
// (src/distributed/tensor_parallel.py:64-84 RMSNorm, :389-419 rotary embedding, :438-462 their
// use in forward), followed by the cache write of the inference path
// (src/inference/attention.py:44-183, called from PagedAttention.forward :225-232):
//
//     q = q_norm(q); k = k_norm(k)                    y = w * (x * rsqrt(mean(x^2) + eps)), fp32, cast back
//     q = rope(q, pos); k = rope(k, pos)              [x1, x2] -> [x1 cos - x2 sin, x2 cos + x1 sin]
//     store_kv_cache(k, v, k_cache, v_cache, slot_mapping, ...)
//
// As separate ops that is some fourteen launches and six round trips of q and k through HBM per
// layer; a decode step touches 64 tokens, so all of it is launch latency.  Here one workgroup
// (8 waves) owns one token: each wave normalises and rotates whole head rows (a lane holds the rotation
// pair i, i + D/2, so the rotation needs no exchange), the rotated K row is collected in LDS so
// that the fp8 writer can take its per-token amax over all heads, and K and V go to their cache
// slot from there.  Intermediate roundings are those of the separate ops: the norm result is
// rounded to the activation dtype, the rotation is done in fp32 on that and rounded again, and
// the fp8 writer sees exactly the values a separate store would see.
#include "pa_common.hpp"
#include "pa_host.hpp"

#include <math.h>

namespace pa {

struct NormRopeParams {
  const void* q;
  const void* k;
  const void* v;
  int64_t q_stride, k_stride, v_stride;   // token strides, elements
  const void* q_weight;
  const void* k_weight;
  const float* inv_freq;                  // [D / 2]
  const int64_t* positions;               // [tokens]
  void* q_out;
  int64_t q_out_stride;
  void* k_out;                            // optional dense copy of the rotated K, may be null
  int64_t k_out_stride;
  uint8_t* k_cache;                       // may be null: no cache write
  uint8_t* v_cache;
  float* k_scale;
  float* v_scale;
  const int32_t* slot_mapping;
  int64_t total_slots;
  int dtype;                              // q, k, v, q_out, k_out (and the cache, unless fp8)
  int weight_dtype;
  int hq, hkv;
  float eps;
};

constexpr int kMaxRow = 4096;  // kv_heads * head_dim that fits the LDS staging row
constexpr int kNormWaves = 8;  // waves per token: 24 head rows at the 16q/8kv shape, three per wave
constexpr int kNormThreads = 64 * kNormWaves;

__device__ __forceinline__ float round_to_dtype(float x, int dtype) {
  if (dtype == PA_DTYPE_F16) return f16_bits_to_f32(f32_to_f16_bits(x));
  if (dtype == PA_DTYPE_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(x));
  return x;
}

__device__ __forceinline__ float nan_keeping_max(float m, float a) { return (a > m || a != a) ? a : m; }

// amax of the workgroup's values -> clamp -> scale, as the quantising store computes them
__device__ __forceinline__ float block_scale(float amax, float* red, int wave, int lane) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = nan_keeping_max(amax, __shfl_xor(amax, o));
  __syncthreads();                       // red may still be read from the previous use
  if (lane == 0) red[wave] = amax;
  __syncthreads();
  amax = red[0];
#pragma unroll
  for (int w = 1; w < kNormWaves; ++w) amax = nan_keeping_max(amax, red[w]);
  amax = amax < 1e-5f ? 1e-5f : amax;    // clamp(min=1e-5); NaN stays NaN
  return __fmul_rn(__fdiv_rn(1.0f, amax), 448.0f);   // torch: amax.reciprocal() * 448
}


// sin and cos of an fp32 angle that may be tens of thousands of radians (position x frequency).
// The reduction to one revolution is done in fp64, where the product with 1/2pi is exact to far
// below an fp32 ulp of the angle; the hardware sine / cosine then take the fraction of a turn.
__device__ __forceinline__ void sincos_turns(float angle, float& sn, float& cs) {
  double turns = (double)angle * 0.15915494309189535;
  turns -= floor(turns);
  const float f = (float)turns;
  sn = __builtin_amdgcn_sinf(f);
  cs = __builtin_amdgcn_cosf(f);
}

template <int D, bool FP8>
__global__ __launch_bounds__(kNormThreads) void qk_norm_rope_store_kernel(const NormRopeParams p) {
  constexpr int HALF = D / 2;
  __shared__ __align__(16) uint16_t krow[kMaxRow];   // rotated K of this token, activation dtype bits
  __shared__ float red[kNormWaves];

  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int es = p.dtype == PA_DTYPE_F32 ? 4 : 2;
  const bool active = lane < HALF;
  const int i = active ? lane : 0;

  const float qw1 = load_as_f32(p.q_weight, i, p.weight_dtype), qw2 = load_as_f32(p.q_weight, i + HALF, p.weight_dtype);
  const float kw1 = load_as_f32(p.k_weight, i, p.weight_dtype), kw2 = load_as_f32(p.k_weight, i + HALF, p.weight_dtype);

  // Every head row of this wave is requested before any is worked on: the rows are independent
  // and a wave that waits for one load at a time spends its life in memory latency.
  constexpr int kRowsPerWave = 4;          // up to 32 head rows per token with 8 waves
  const int nrows = p.hq + p.hkv;
  float xa[kRowsPerWave], xb[kRowsPerWave];
#pragma unroll
  for (int j = 0; j < kRowsPerWave; ++j) {
    const int r = wave + j * kNormWaves;
    xa[j] = xb[j] = 0.0f;
    if (active && r < nrows) {
      const bool is_k = r >= p.hq;
      const int64_t base = t * (is_k ? p.k_stride : p.q_stride) + (int64_t)(is_k ? r - p.hq : r) * D;
      xa[j] = load_as_f32(is_k ? p.k : p.q, base + i, p.dtype);
      xb[j] = load_as_f32(is_k ? p.k : p.q, base + i + HALF, p.dtype);
    }
  }
  float cs, sn;
  sincos_turns((float)p.positions[t] * p.inv_freq[i], sn, cs);
#pragma unroll
  for (int j = 0; j < kRowsPerWave; ++j) {
    const int r = wave + j * kNormWaves;
    if (r >= nrows) break;                 // wave-uniform
    const bool is_k = r >= p.hq;
    const int head = is_k ? r - p.hq : r;
    const float x1 = xa[j], x2 = xb[j];
    float ss = x1 * x1 + x2 * x2;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    const float inv = rsqrtf(ss / (float)D + p.eps);
    // the norm returns the activation dtype; the rotation then works in fp32 on those values
    const float y1 = round_to_dtype((is_k ? kw1 : qw1) * (x1 * inv), p.dtype);
    const float y2 = round_to_dtype((is_k ? kw2 : qw2) * (x2 * inv), p.dtype);
    const float o1 = y1 * cs + (-y2) * sn;
    const float o2 = y2 * cs + y1 * sn;
    if (!active) continue;
    if (!is_k) {
      const int64_t ob = t * p.q_out_stride + (int64_t)head * D;
      store_from_f32(p.q_out, ob + i, p.dtype, o1);
      store_from_f32(p.q_out, ob + i + HALF, p.dtype, o2);
    } else {
      if (p.k_out) {
        const int64_t ob = t * p.k_out_stride + (int64_t)head * D;
        store_from_f32(p.k_out, ob + i, p.dtype, o1);
        store_from_f32(p.k_out, ob + i + HALF, p.dtype, o2);
      }
      if (p.dtype == PA_DTYPE_F32) {
        ((float*)krow)[head * D + i] = o1;          // fp32 activations: the row is kMaxRow / 2 long at most
        ((float*)krow)[head * D + i + HALF] = o2;
      } else {
        krow[head * D + i] = p.dtype == PA_DTYPE_F16 ? f32_to_f16_bits(o1) : f32_to_bf16_bits(o1);
        krow[head * D + i + HALF] = p.dtype == PA_DTYPE_F16 ? f32_to_f16_bits(o2) : f32_to_bf16_bits(o2);
      }
    }
  }
  __syncthreads();

  if (!p.k_cache) return;
  const int64_t slot = p.slot_mapping[t];
  if (slot < 0 || slot >= p.total_slots) return;   // uniform over the workgroup
  const int row = p.hkv * D;
  const uint8_t* vsrc = (const uint8_t*)p.v + t * p.v_stride * es;

  if constexpr (!FP8) {
    // same-dtype cache: 16-byte pieces of the staged K row and of the V row
    const int64_t row_bytes = (int64_t)row * es;
    uint8_t* kd = p.k_cache + slot * row_bytes;
    uint8_t* vd = p.v_cache + slot * row_bytes;
    for (int64_t off = (int64_t)threadIdx.x * 16; off < row_bytes; off += kNormThreads * 16) {
      *(uint4*)(kd + off) = *(const uint4*)((const uint8_t*)krow + off);
      *(uint4*)(vd + off) = *(const uint4*)(vsrc + off);
    }
  } else {
    // quantising cache: per-token amax over all heads, scale = (1/amax) * 448, e4m3fn bytes
    auto quantise = [&](const void* src_row, uint8_t* dst, float* scale_dst) {
      float amax = 0.0f;
      for (int e = threadIdx.x * 8; e < row; e += kNormThreads * 8) {
        float x[8];
        load8_as_f32(src_row, e, p.dtype, x);
#pragma unroll
        for (int j = 0; j < 8; ++j) amax = nan_keeping_max(amax, fabsf(x[j]));
      }
      const float s = block_scale(amax, red, wave, lane);
      if (threadIdx.x == 0) *scale_dst = s;
      for (int e = threadIdx.x * 8; e < row; e += kNormThreads * 8) {
        float x[8];
        load8_as_f32(src_row, e, p.dtype, x);
        uint32_t w[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          uint32_t b = 0;
#pragma unroll
          for (int k = 0; k < 4; ++k) b |= f32_to_e4m3fn(__fmul_rn(x[4 * j + k], s)) << (8 * k);
          w[j] = b;
        }
        *(uint2*)(dst + e) = make_uint2(w[0], w[1]);
      }
    };
    quantise(krow, p.k_cache + slot * row, p.k_scale + slot);
    quantise(vsrc, p.v_cache + slot * row, p.v_scale + slot);
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_qk_norm_rope_store(const void* q, const void* k, const void* v, int dtype, int64_t q_token_stride,
                                     int64_t k_token_stride, int64_t v_token_stride, const void* q_norm_weight,
                                     const void* k_norm_weight, int weight_dtype, float eps, const float* inv_freq,
                                     const int64_t* positions, void* q_out, int64_t q_out_token_stride, void* k_out,
                                     int64_t k_out_token_stride, void* k_cache, void* v_cache, float* k_scale,
                                     float* v_scale, int kv_dtype, const int32_t* slot_mapping, int64_t num_tokens,
                                     int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t total_slots,
                                     void* stream) {
  if (num_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_qk_norm_rope_store: negative or zero size");
  if (num_tokens == 0) return PA_OK;
  if (!q || !k || !q_norm_weight || !k_norm_weight || !inv_freq || !positions || !q_out)
    return fail(PA_ERR_BAD_ARG, "pa_qk_norm_rope_store: null pointer");
  if (dtype != PA_DTYPE_F16 && dtype != PA_DTYPE_BF16 && dtype != PA_DTYPE_F32)
    return fail(PA_ERR_UNSUPPORTED, "pa_qk_norm_rope_store: dtype must be f16, bf16 or f32");
  if (weight_dtype != PA_DTYPE_F16 && weight_dtype != PA_DTYPE_BF16 && weight_dtype != PA_DTYPE_F32)
    return fail(PA_ERR_UNSUPPORTED, "pa_qk_norm_rope_store: weight_dtype must be f16, bf16 or f32");
  if (head_dim != 64 && head_dim != 128)
    return fail(PA_ERR_UNSUPPORTED, "pa_qk_norm_rope_store: head_dim must be 64 or 128");
  const int es = dtype == PA_DTYPE_F32 ? 4 : 2;
  if (num_kv_heads * head_dim * es > kMaxRow * 2)
    return fail(PA_ERR_UNSUPPORTED, "pa_qk_norm_rope_store: kv_heads * head_dim too large for the staging row");
  if (q_token_stride < num_q_heads * head_dim || q_out_token_stride < num_q_heads * head_dim ||
      k_token_stride < num_kv_heads * head_dim || (k_out && k_out_token_stride < num_kv_heads * head_dim))
    return fail(PA_ERR_BAD_ARG, "pa_qk_norm_rope_store: token stride smaller than a row");
  const bool fp8 = kv_dtype == PA_DTYPE_FP8_E4M3;
  if (k_cache) {
    if (!v || !v_cache || !slot_mapping || total_slots <= 0)
      return fail(PA_ERR_BAD_ARG, "pa_qk_norm_rope_store: the cache write needs v, v_cache, slot_mapping and total_slots");
    if (!fp8 && kv_dtype != dtype)
      return fail(PA_ERR_UNSUPPORTED, "pa_qk_norm_rope_store: cache dtype must be the activation dtype or fp8-e4m3");
    if (fp8 && (!k_scale || !v_scale))
      return fail(PA_ERR_BAD_ARG, "pa_qk_norm_rope_store: fp8 cache needs k_scale and v_scale");
    if (v_token_stride < num_kv_heads * head_dim || (v_token_stride * es) % 16 != 0 || !aligned16(v) ||
        !aligned16(k_cache) || !aligned16(v_cache))
      return fail(PA_ERR_BAD_ARG, "pa_qk_norm_rope_store: v rows and caches must be 16-byte aligned");
  }
  if (num_tokens > 0x7fffffff) return fail(PA_ERR_UNSUPPORTED, "pa_qk_norm_rope_store: too many tokens");
  if (num_q_heads + num_kv_heads > 4 * kNormWaves)
    return fail(PA_ERR_UNSUPPORTED, "pa_qk_norm_rope_store: more than 32 q + kv heads per token");

  NormRopeParams p;
  p.q = q; p.k = k; p.v = v;
  p.q_stride = q_token_stride; p.k_stride = k_token_stride; p.v_stride = v_token_stride;
  p.q_weight = q_norm_weight; p.k_weight = k_norm_weight;
  p.inv_freq = inv_freq; p.positions = positions;
  p.q_out = q_out; p.q_out_stride = q_out_token_stride;
  p.k_out = k_out; p.k_out_stride = k_out_token_stride;
  p.k_cache = (uint8_t*)k_cache; p.v_cache = (uint8_t*)v_cache;
  p.k_scale = k_scale; p.v_scale = v_scale;
  p.slot_mapping = slot_mapping; p.total_slots = total_slots;
  p.dtype = dtype; p.weight_dtype = weight_dtype;
  p.hq = (int)num_q_heads; p.hkv = (int)num_kv_heads;
  p.eps = eps;

  dim3 grid((unsigned)num_tokens);
  hipStream_t st = (hipStream_t)stream;
  if (head_dim == 128) {
    if (fp8) hipLaunchKernelGGL((qk_norm_rope_store_kernel<128, true>), grid, dim3(kNormThreads), 0, st, p);
    else hipLaunchKernelGGL((qk_norm_rope_store_kernel<128, false>), grid, dim3(kNormThreads), 0, st, p);
  } else {
    if (fp8) hipLaunchKernelGGL((qk_norm_rope_store_kernel<64, true>), grid, dim3(kNormThreads), 0, st, p);
    else hipLaunchKernelGGL((qk_norm_rope_store_kernel<64, false>), grid, dim3(kNormThreads), 0, st, p);
  }
  return check_launch("pa_qk_norm_rope_store");
}
