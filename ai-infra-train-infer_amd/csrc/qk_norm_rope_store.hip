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
// layer; a decode step touches 64 tokens, so all of it is launch latency.  Here one wave owns
// one token and nothing leaves its registers: a lane holds 8 consecutive elements of a head row
// (16-byte accesses; 16 lanes per row at head_dim 128, so one instruction covers four heads), the
// rotation partner of an element sits 8 lanes away (one cross-lane move), RMSNorm needs a
// 16-lane sum, and the per-token amax of the fp8 writer is a wave reduction over the rotated K
// rows the wave still holds.  Intermediate roundings are those of the separate ops: the norm
// result is rounded to the activation dtype, the rotation is done in fp32 on that and rounded
// again, and the fp8 writer sees exactly the values a separate store would see.
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
  int64_t num_tokens;
  int dtype;                              // q, k, v, q_out, k_out (and the cache, unless fp8)
  int weight_dtype;
  int hq, hkv;
  float eps;
};

constexpr int kTokensPerGroup = 4;   // waves (= tokens) per workgroup
constexpr int kMaxKvGroups = 4;      // K row groups a wave keeps in registers: kv_heads * head_dim <= 2048
// Launches of up to this many tokens run one wave per (token, row group): 64 tokens 5.5 -> 3.7 us inside a
// replayed graph, 512 tokens 6.0 -> 5.3; from 1024 tokens on the token-per-wave kernel is the faster one
// (the angles are worked out once per token instead of once per row group).
constexpr int64_t kSplitUpToTokens = 512;

__device__ __forceinline__ float round_to_dtype(float x, int dtype) {
  if (dtype == PA_DTYPE_F16) return f16_bits_to_f32(f32_to_f16_bits(x));
  if (dtype == PA_DTYPE_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(x));
  return x;
}

__device__ __forceinline__ float nan_keeping_max(float m, float a) { return (a > m || a != a) ? a : m; }

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

// eight consecutive elements (index i a multiple of 8, 16-byte aligned rows) from fp32
__device__ __forceinline__ void store8_from_f32(void* p, int64_t i, int dtype, const float (&x)[8]) {
  if (dtype == PA_DTYPE_F32) {
    *(float4*)((float*)p + i) = make_float4(x[0], x[1], x[2], x[3]);
    *(float4*)((float*)p + i + 4) = make_float4(x[4], x[5], x[6], x[7]);
  } else {
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t lo = dtype == PA_DTYPE_F16 ? f32_to_f16_bits(x[2 * k]) : f32_to_bf16_bits(x[2 * k]);
      const uint32_t hi = dtype == PA_DTYPE_F16 ? f32_to_f16_bits(x[2 * k + 1]) : f32_to_bf16_bits(x[2 * k + 1]);
      w[k] = lo | (hi << 16);
    }
    *(uint4*)((uint16_t*)p + i) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

// amax over the wave -> clamp -> scale, as the quantising store computes them
__device__ __forceinline__ float wave_scale(float amax) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = nan_keeping_max(amax, __shfl_xor(amax, o));
  amax = amax < 1e-5f ? 1e-5f : amax;    // clamp(min=1e-5); NaN stays NaN
  return __fmul_rn(__fdiv_rn(1.0f, amax), 448.0f);   // torch: amax.reciprocal() * 448
}

__device__ __forceinline__ uint2 encode8(const float (&x)[8], float s) {
  uint32_t w[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    // the hardware conversion, as in kv_store_fp8_kernel (same bytes on the range the scale allows)
    int b = 0;
    b = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(x[4 * j], s), __fmul_rn(x[4 * j + 1], s), b, false);
    b = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(x[4 * j + 2], s), __fmul_rn(x[4 * j + 3], s), b, true);
    w[j] = (uint32_t)b;
  }
  return make_uint2(w[0], w[1]);
}

// DT = activation dtype, a template parameter: a run-time switch inside every 8-element load and
// store would put a branch (and a wait) between the loads that are meant to be in flight together.
template <int D, bool FP8, int DT>
__global__ __launch_bounds__(64 * kTokensPerGroup) void qk_norm_rope_store_kernel(const NormRopeParams p) {
  constexpr int LPR = D / 8;          // lanes per head row
  constexpr int RPI = 64 / LPR;       // head rows per wave instruction
  constexpr int PAIR = LPR / 2;       // lane distance to the rotation partner
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * kTokensPerGroup + (threadIdx.x >> 6);
  if (t >= p.num_tokens) return;      // the whole wave
  const int c = lane % LPR;           // which 8 elements of the row
  const int sub = lane / LPR;         // which row of the group
  const bool upper = c >= PAIR;       // second half of the row
  const int f0 = (c % PAIR) * 8;      // first of this lane's 8 frequencies

  // loads first, all of them: position, frequencies, weights and (below) every row of the token
  const float pos = (float)p.positions[t];
  const float4 fa = *(const float4*)(p.inv_freq + f0), fb = *(const float4*)(p.inv_freq + f0 + 4);
  float qw[8], kw[8];
  load8_as_f32(p.q_weight, c * 8, p.weight_dtype, qw);
  load8_as_f32(p.k_weight, c * 8, p.weight_dtype, kw);
  // Every row group of the token is requested before any is worked on: they are independent,
  // and a wave that waits for one load at a time spends its life in memory latency.
  constexpr int kQGroupsAhead = 4;      // q row groups loaded up front (16 heads at head_dim 128)
  float qx[kQGroupsAhead][8], kx[kMaxKvGroups][8], vx[kMaxKvGroups][8];
#pragma unroll
  for (int g = 0; g < kQGroupsAhead; ++g) {
    const int head = g * RPI + sub;
#pragma unroll
    for (int e = 0; e < 8; ++e) qx[g][e] = 0.0f;
    if (head < p.hq) load8_as_f32(p.q, t * p.q_stride + (int64_t)head * D + c * 8, DT, qx[g]);
  }
  const bool write = p.k_cache != nullptr;
  const int64_t slot = write ? (int64_t)p.slot_mapping[t] : -1;
#pragma unroll
  for (int g = 0; g < kMaxKvGroups; ++g) {
    const int head = g * RPI + sub;
#pragma unroll
    for (int e = 0; e < 8; ++e) kx[g][e] = vx[g][e] = 0.0f;
    if (head < p.hkv) {
      load8_as_f32(p.k, t * p.k_stride + (int64_t)head * D + c * 8, DT, kx[g]);
      if (write) load8_as_f32(p.v, t * p.v_stride + (int64_t)head * D + c * 8, DT, vx[g]);
    }
  }

  float cs[8], sn[8];
  {
    const float fr[8] = {fa.x, fa.y, fa.z, fa.w, fb.x, fb.y, fb.z, fb.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) sincos_turns(pos * fr[e], sn[e], cs[e]);
  }

  // x: this lane's 8 elements of a head row -> normalised, rounded, rotated, rounded (as fp32)
  auto norm_rope = [&](float (&x)[8], const float (&w)[8]) __attribute__((always_inline)) {
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
    // sum over the LPR lanes of the row, by lane-permute moves inside a 16-lane row
    ss += dpp_f32<0xB1>(ss);                        // quad_perm [1,0,3,2]
    ss += dpp_f32<0x4E>(ss);                        // quad_perm [2,3,0,1]
    if constexpr (LPR == 16) {
      ss += dpp_f32<0x124>(ss);                     // row_ror:4
      ss += dpp_f32<0x128>(ss);                     // row_ror:8
    } else {
      ss += dpp_f32<0x141>(ss);                     // row_half_mirror: lane i <-> 7 - i
    }
    const float inv = rsqrtf(ss / (float)D + p.eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      // the norm returns the activation dtype; the rotation then works in fp32 on those values
      const float y = round_to_dtype(w[e] * (x[e] * inv), DT);
      // the rotation partner: 8 lanes away in a 16-lane row (row_ror:8), 4 away in an 8-lane one
      const float other = LPR == 16 ? dpp_f32<0x128>(y) : __shfl_xor(y, PAIR);
      const float rotated = upper ? other : -other;      // cat(-x2, x1)
      x[e] = round_to_dtype(y * cs[e] + rotated * sn[e], DT);
    }
  };

  // ---- q ------------------------------------------------------------------------------------------
#pragma unroll
  for (int g = 0; g < kQGroupsAhead; ++g) {
    const int head = g * RPI + sub;
    if (g * RPI < p.hq) {                // wave-uniform
      norm_rope(qx[g], qw);
      if (head < p.hq) store8_from_f32(p.q_out, t * p.q_out_stride + (int64_t)head * D + c * 8, DT, qx[g]);
    }
  }
  for (int g = kQGroupsAhead; g * RPI < p.hq; ++g) {      // more query heads than were loaded up front
    const int head = g * RPI + sub;
    const bool live = head < p.hq;
    float x[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (live) load8_as_f32(p.q, t * p.q_stride + (int64_t)head * D + c * 8, DT, x);
    norm_rope(x, qw);
    if (live) store8_from_f32(p.q_out, t * p.q_out_stride + (int64_t)head * D + c * 8, DT, x);
  }

  // ---- k: the rotated rows stay in registers for the cache write -------------------------------------
#pragma unroll
  for (int g = 0; g < kMaxKvGroups; ++g) {
    const int head = g * RPI + sub;
    if (g * RPI < p.hkv) {               // wave-uniform
      norm_rope(kx[g], kw);
      if (head < p.hkv && p.k_out)
        store8_from_f32(p.k_out, t * p.k_out_stride + (int64_t)head * D + c * 8, DT, kx[g]);
    }
  }

  // ---- cache write ----------------------------------------------------------------------------------
  if (!write || slot < 0 || slot >= p.total_slots) return;   // uniform over the wave
  const int64_t row = (int64_t)p.hkv * D;
  if constexpr (!FP8) {
#pragma unroll
    for (int g = 0; g < kMaxKvGroups; ++g) {
      const int head = g * RPI + sub;
      if (head < p.hkv) {
        store8_from_f32(p.k_cache, slot * row + (int64_t)head * D + c * 8, DT, kx[g]);
        store8_from_f32(p.v_cache, slot * row + (int64_t)head * D + c * 8, DT, vx[g]);
      }
    }
  } else {
    // per-token amax over all heads, scale = (1/amax) * 448, e4m3fn bytes; rows of dead lanes are zero
    float ka = 0.0f, va = 0.0f;
#pragma unroll
    for (int g = 0; g < kMaxKvGroups; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        ka = nan_keeping_max(ka, fabsf(kx[g][e]));
        va = nan_keeping_max(va, fabsf(vx[g][e]));
      }
    const float ksc = wave_scale(ka), vsc = wave_scale(va);
    if (lane == 0) {
      p.k_scale[slot] = ksc;
      p.v_scale[slot] = vsc;
    }
#pragma unroll
    for (int g = 0; g < kMaxKvGroups; ++g) {
      const int head = g * RPI + sub;
      if (head < p.hkv) {
        *(uint2*)(p.k_cache + slot * row + (int64_t)head * D + c * 8) = encode8(kx[g], ksc);
        *(uint2*)(p.v_cache + slot * row + (int64_t)head * D + c * 8) = encode8(vx[g], vsc);
      }
    }
  }
}


// The same work cut finer, for launches of few tokens (a decode step): one wave per (token, row
// group) - a wave for each group of 64 / (head_dim / 8) query heads, one more for the token's K and V
// rows (the fp8 writer's per-token amax runs over all K heads, so those stay in one wave).  A
// decode step's 64 tokens then run as 320 short waves over 80 CUs instead of 64 long ones over 16,
// and a wave's program is a sixth as long: straight-line code that runs once is fetched from
// memory as it goes, which is most of what a launch of this size lasts.  Element for element the
// arithmetic is the kernel's above.
template <int D, bool FP8, int DT>
__global__ __launch_bounds__(64 * kTokensPerGroup) void qk_norm_rope_store_split_kernel(const NormRopeParams p,
                                                                                        const int q_groups) {
  constexpr int LPR = D / 8;
  constexpr int RPI = 64 / LPR;
  constexpr int PAIR = LPR / 2;
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * kTokensPerGroup + (threadIdx.x >> 6);
  const int roles = q_groups + 1;
  const int64_t t = w / roles;
  const int role = __builtin_amdgcn_readfirstlane((int)(w % roles));   // < q_groups: that group of q rows; else K and V
  if (t >= p.num_tokens) return;      // the whole wave
  const int c = lane % LPR;
  const int sub = lane / LPR;
  const bool upper = c >= PAIR;
  const int f0 = (c % PAIR) * 8;
  const bool is_q = role < q_groups;

  const float pos = (float)p.positions[t];
  const float4 fa = *(const float4*)(p.inv_freq + f0), fb = *(const float4*)(p.inv_freq + f0 + 4);
  float wt[8], x[kMaxKvGroups][8], vx[kMaxKvGroups][8];
#pragma unroll
  for (int g = 0; g < kMaxKvGroups; ++g)
#pragma unroll
    for (int e = 0; e < 8; ++e) x[g][e] = vx[g][e] = 0.0f;
  const bool write = p.k_cache != nullptr;
  int64_t slot = -1;
  if (is_q) {
    load8_as_f32(p.q_weight, c * 8, p.weight_dtype, wt);
    const int head = role * RPI + sub;
    if (head < p.hq) load8_as_f32(p.q, t * p.q_stride + (int64_t)head * D + c * 8, DT, x[0]);
  } else {
    load8_as_f32(p.k_weight, c * 8, p.weight_dtype, wt);
    if (write) slot = (int64_t)p.slot_mapping[t];
#pragma unroll
    for (int g = 0; g < kMaxKvGroups; ++g) {
      const int head = g * RPI + sub;
      if (head < p.hkv) {
        load8_as_f32(p.k, t * p.k_stride + (int64_t)head * D + c * 8, DT, x[g]);
        if (write) load8_as_f32(p.v, t * p.v_stride + (int64_t)head * D + c * 8, DT, vx[g]);
      }
    }
  }

  float cs[8], sn[8];
  {
    const float fr[8] = {fa.x, fa.y, fa.z, fa.w, fb.x, fb.y, fb.z, fb.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) sincos_turns(pos * fr[e], sn[e], cs[e]);
  }

  // one row group: the loop below runs once for a q wave, once per K row group for the other
  const int groups = is_q ? 1 : (p.hkv + RPI - 1) / RPI;
#pragma unroll
  for (int g = 0; g < kMaxKvGroups; ++g) {
    if (g >= groups) continue;         // wave-uniform
    float (&r)[8] = x[g];
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += r[e] * r[e];
    ss += dpp_f32<0xB1>(ss);
    ss += dpp_f32<0x4E>(ss);
    if constexpr (LPR == 16) {
      ss += dpp_f32<0x124>(ss);
      ss += dpp_f32<0x128>(ss);
    } else {
      ss += dpp_f32<0x141>(ss);
    }
    const float inv = rsqrtf(ss / (float)D + p.eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float y = round_to_dtype(wt[e] * (r[e] * inv), DT);
      const float other = LPR == 16 ? dpp_f32<0x128>(y) : __shfl_xor(y, PAIR);
      const float rotated = upper ? other : -other;
      r[e] = round_to_dtype(y * cs[e] + rotated * sn[e], DT);
    }
  }

  if (is_q) {
    const int head = role * RPI + sub;
    if (head < p.hq) store8_from_f32(p.q_out, t * p.q_out_stride + (int64_t)head * D + c * 8, DT, x[0]);
    return;
  }
  if (p.k_out) {
#pragma unroll
    for (int g = 0; g < kMaxKvGroups; ++g) {
      const int head = g * RPI + sub;
      if (head < p.hkv) store8_from_f32(p.k_out, t * p.k_out_stride + (int64_t)head * D + c * 8, DT, x[g]);
    }
  }
  if (!write || slot < 0 || slot >= p.total_slots) return;   // uniform over the wave
  const int64_t row = (int64_t)p.hkv * D;
  if constexpr (!FP8) {
#pragma unroll
    for (int g = 0; g < kMaxKvGroups; ++g) {
      const int head = g * RPI + sub;
      if (head < p.hkv) {
        store8_from_f32(p.k_cache, slot * row + (int64_t)head * D + c * 8, DT, x[g]);
        store8_from_f32(p.v_cache, slot * row + (int64_t)head * D + c * 8, DT, vx[g]);
      }
    }
  } else {
    float ka = 0.0f, va = 0.0f;
#pragma unroll
    for (int g = 0; g < kMaxKvGroups; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        ka = nan_keeping_max(ka, fabsf(x[g][e]));
        va = nan_keeping_max(va, fabsf(vx[g][e]));
      }
    const float ksc = wave_scale(ka), vsc = wave_scale(va);
    if (lane == 0) {
      p.k_scale[slot] = ksc;
      p.v_scale[slot] = vsc;
    }
#pragma unroll
    for (int g = 0; g < kMaxKvGroups; ++g) {
      const int head = g * RPI + sub;
      if (head < p.hkv) {
        *(uint2*)(p.k_cache + slot * row + (int64_t)head * D + c * 8) = encode8(x[g], ksc);
        *(uint2*)(p.v_cache + slot * row + (int64_t)head * D + c * 8) = encode8(vx[g], vsc);
      }
    }
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
  if (num_kv_heads * head_dim > kMaxKvGroups * 512)
    return fail(PA_ERR_UNSUPPORTED, "pa_qk_norm_rope_store: kv_heads * head_dim must not exceed 2048");
  // every row is moved in 16-byte pieces
  const auto rows16 = [&](const void* base, int64_t stride) { return aligned16(base) && (stride * es) % 16 == 0; };
  if (!rows16(q, q_token_stride) || !rows16(k, k_token_stride) || !rows16(q_out, q_out_token_stride) ||
      (k_out && !rows16(k_out, k_out_token_stride)) || !aligned16(q_norm_weight) || !aligned16(k_norm_weight) ||
      !aligned16(inv_freq))
    return fail(PA_ERR_BAD_ARG, "pa_qk_norm_rope_store: rows, weights and inv_freq must be 16-byte aligned");
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
  p.num_tokens = num_tokens;
  p.dtype = dtype; p.weight_dtype = weight_dtype;
  p.hq = (int)num_q_heads; p.hkv = (int)num_kv_heads;
  p.eps = eps;

  dim3 grid((unsigned)((num_tokens + kTokensPerGroup - 1) / kTokensPerGroup));
  hipStream_t st = (hipStream_t)stream;
  // few tokens: one wave per (token, row group) instead of one per token
  const int rows_per_wave = 64 / ((int)head_dim / 8);
  const int q_groups = ((int)num_q_heads + rows_per_wave - 1) / rows_per_wave;
  const bool split = num_tokens <= kSplitUpToTokens;
  if (split) grid = dim3((unsigned)((num_tokens * (q_groups + 1) + kTokensPerGroup - 1) / kTokensPerGroup));
#define PA_LAUNCH_NORM_ROPE(DIM, F8, DT)                                                                         \
  if (split)                                                                                                     \
    hipLaunchKernelGGL((qk_norm_rope_store_split_kernel<DIM, F8, DT>), grid, dim3(64 * kTokensPerGroup), 0, st, p, \
                       q_groups);                                                                                \
  else                                                                                                           \
    hipLaunchKernelGGL((qk_norm_rope_store_kernel<DIM, F8, DT>), grid, dim3(64 * kTokensPerGroup), 0, st, p)
#define PA_LAUNCH_NORM_ROPE_DT(DIM, F8)                                  \
  switch (dtype) {                                                       \
    case PA_DTYPE_F16: PA_LAUNCH_NORM_ROPE(DIM, F8, PA_DTYPE_F16); break;   \
    case PA_DTYPE_BF16: PA_LAUNCH_NORM_ROPE(DIM, F8, PA_DTYPE_BF16); break; \
    default: PA_LAUNCH_NORM_ROPE(DIM, F8, PA_DTYPE_F32); break;             \
  }
  if (head_dim == 128) {
    if (fp8) { PA_LAUNCH_NORM_ROPE_DT(128, true) } else { PA_LAUNCH_NORM_ROPE_DT(128, false) }
  } else {
    if (fp8) { PA_LAUNCH_NORM_ROPE_DT(64, true) } else { PA_LAUNCH_NORM_ROPE_DT(64, false) }
  }
#undef PA_LAUNCH_NORM_ROPE_DT
#undef PA_LAUNCH_NORM_ROPE
  return check_launch("pa_qk_norm_rope_store");
}
