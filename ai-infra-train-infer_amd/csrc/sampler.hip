// Token sampling from a batch of logit rows on the GPU (gfx950): greedy argmax, or temperature +
// nucleus (top-p) sampling.
//
// Reference: ModelRunner.sample (src/inference/model_runner.py:590-634):
//     temperature <= 0:  argmax(logits)
//     otherwise:         scaled = logits.float() / temperature
//                        top_p < 1: sort descending, softmax, cumulative sum; a token stays iff the
//                        mass of the tokens ranked before it is <= top_p (the first always stays)
//                        probs = softmax(scaled restricted to the kept tokens); draw one token
// which costs a full sort of the vocabulary, a scatter back and a multinomial per step, and ends
// in .tolist() (a host synchronisation).
//
// Here one workgroup owns one row and never sorts.  "The mass ranked before token j" is
// G(l_j) = sum of p_i over logits l_i > l_j, and G is monotone in the logit, so the kept set is
// {j : l_j >= t*} with t* the smallest logit whose G is <= top_p: t* is found by bisection over the
// ordered bit patterns of the logit type (16 passes for fp16 / bf16 rows, 32 for fp32) with the
// row resident in L2.  The draw itself is an inverse-CDF lookup in index order with a uniform
// number supplied by the caller, so a step is reproducible and needs no generator state on the
// device: the first index j with sum_{i <= j, kept} p_i > u * (kept mass).
// Logits tied with t* all stay (a sort keeps an implementation-defined subset of such a tie).
#include "pa_common.hpp"
#include "pa_host.hpp"

#include <math.h>

namespace pa {

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / 64;

// bit pattern -> unsigned key with the same order as the float value (-0 < +0 is harmless here)
__device__ __forceinline__ uint32_t ordered_key32(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ uint32_t ordered_key16(uint32_t h) {
  return (h & 0x8000u) ? (~h & 0xffffu) : (h | 0x8000u);
}

template <int DT>
struct Row {
  const void* p;
  __device__ __forceinline__ float value(int64_t i) const {
    if constexpr (DT == PA_DTYPE_F32) return ((const float*)p)[i];
    else if constexpr (DT == PA_DTYPE_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
    else return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  }
  // order-preserving key: 32 bits for fp32 rows, 16 for the 16-bit types
  __device__ __forceinline__ uint32_t key(int64_t i) const {
    if constexpr (DT == PA_DTYPE_F32) return ordered_key32(((const float*)p)[i]);
    else return ordered_key16(((const uint16_t*)p)[i]);
  }
  __device__ __forceinline__ static float bits_value(uint32_t bits) {
    if constexpr (DT == PA_DTYPE_F32) return __uint_as_float(bits);
    else if constexpr (DT == PA_DTYPE_F16) return f16_bits_to_f32(bits);
    else return bf16_bits_to_f32(bits);
  }
  __device__ __forceinline__ static uint32_t bits_key(uint32_t bits) {
    if constexpr (DT == PA_DTYPE_F32) return ordered_key32(__uint_as_float(bits));
    else return ordered_key16(bits);
  }
  // f(index, raw bits) for every element of the row, the workgroup's threads taking 16-byte
  // pieces in turn (scalar accesses when the row is not 16-byte aligned, and for the tail)
  template <class F>
  __device__ __forceinline__ void for_each(int64_t vocab, F&& f) const {
    constexpr int PER = DT == PA_DTYPE_F32 ? 4 : 8;
    const bool wide = (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
    const int64_t nvec = wide ? vocab / PER : 0;
    for (int64_t c = threadIdx.x; c < nvec; c += kSampleThreads) {
      const uint4 w = ((const uint4*)p)[c];
      const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if constexpr (DT == PA_DTYPE_F32) {
          f(c * 4 + k, ww[k]);
        } else {
          f(c * 8 + 2 * k, ww[k] & 0xffffu);
          f(c * 8 + 2 * k + 1, ww[k] >> 16);
        }
      }
    }
    for (int64_t i = nvec * PER + threadIdx.x; i < vocab; i += kSampleThreads) {
      if constexpr (DT == PA_DTYPE_F32) f(i, __float_as_uint(((const float*)p)[i]));
      else f(i, (uint32_t)((const uint16_t*)p)[i]);
    }
  }
};

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.0f;
#pragma unroll
  for (int w = 0; w < kSampleWaves; ++w) s += red[w];   // same order in every thread
  return s;
}

template <int DT>
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(const void* __restrict__ logits, int64_t row_stride,
                                                                int64_t vocab, float temperature, float top_p,
                                                                const float* __restrict__ uniforms,
                                                                int64_t* __restrict__ out) {
  __shared__ float red[kSampleWaves];
  __shared__ float redv[kSampleWaves];
  __shared__ int64_t redi[kSampleWaves];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t b = blockIdx.x;
  Row<DT> row{(const uint8_t*)logits + b * row_stride * (DT == PA_DTYPE_F32 ? 4 : 2)};

  // ---- max and its first index ----------------------------------------------------------------
  float best = -INFINITY;
  int64_t best_i = vocab;     // NaN rows fall through with no index: reported as 0 below
  row.for_each(vocab, [&](int64_t i, uint32_t bits) {
    const float x = Row<DT>::bits_value(bits);
    if (x > best || (x == best && i < best_i)) { best = x; best_i = i; }
  });
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o);
    const int64_t oi = __shfl_xor(best_i, o);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  }
  if (lane == 0) { redv[wave] = best; redi[wave] = best_i; }
  __syncthreads();
  best = redv[0]; best_i = redi[0];
#pragma unroll
  for (int w = 1; w < kSampleWaves; ++w)
    if (redv[w] > best || (redv[w] == best && redi[w] < best_i)) { best = redv[w]; best_i = redi[w]; }
  if (best_i >= vocab) best_i = 0;
  if (temperature <= 0.0f) {
    if (tid == 0) out[b] = best_i;
    return;
  }

  // ---- softmax mass relative to the max: p_i = exp2((l_i - max) * c) / Z ----------------------------
  const float c = 1.4426950408889634f / temperature;
  auto weight = [&](int64_t i) { return exp2f((row.value(i) - best) * c); };
  auto bits_weight = [&](uint32_t bits) { return exp2f((Row<DT>::bits_value(bits) - best) * c); };
  float z = 0.0f;
  row.for_each(vocab, [&](int64_t, uint32_t bits) { z += bits_weight(bits); });
  z = block_sum(z, red);

  // ---- nucleus threshold: smallest key t with mass(key > t) <= top_p * Z ---------------------------
  uint32_t thr = 0;            // keep everything
  if (top_p < 1.0f) {
    constexpr int BITS = DT == PA_DTYPE_F32 ? 32 : 16;
    const float limit = top_p * z;
    // invariant: mass(key > hi) <= limit (true for the largest key), lo - 1 violates it or lo == 0
    uint32_t lo = 0, hi = BITS == 32 ? 0xffffffffu : 0xffffu;
    for (int it = 0; it < BITS; ++it) {
      const uint32_t mid = lo + ((hi - lo) >> 1);
      float above = 0.0f;
      row.for_each(vocab, [&](int64_t, uint32_t bits) {
        if (Row<DT>::bits_key(bits) > mid) above += bits_weight(bits);
      });
      above = block_sum(above, red);
      if (above <= limit) hi = mid; else lo = mid + 1;     // uniform over the workgroup
    }
    thr = hi;
  }

  // ---- inverse CDF in index order over the kept tokens -----------------------------------------------
  // wave w owns the contiguous range [w * span, (w + 1) * span)
  const int64_t span = ((vocab + kSampleWaves - 1) / kSampleWaves + 63) / 64 * 64;
  const int64_t begin = (int64_t)wave * span, end = begin + span < vocab ? begin + span : vocab;
  float mine = 0.0f;
  for (int64_t i = begin + lane; i < end; i += 64)
    if (row.key(i) >= thr) mine += weight(i);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o);
  __syncthreads();
  if (lane == 0) red[wave] = mine;
  __syncthreads();
  float kept = 0.0f;
#pragma unroll
  for (int w = 0; w < kSampleWaves; ++w) kept += red[w];
  const float target = uniforms[b] * kept;
  // the wave in whose range the running sum passes the target (the last non-empty one if rounding
  // leaves the target at or above the total)
  float before = 0.0f;
  int owner = -1, last_nonempty = 0;
#pragma unroll
  for (int w = 0; w < kSampleWaves; ++w) {
    if (red[w] > 0.0f) last_nonempty = w;
    if (owner < 0 && before + red[w] > target) owner = w; else if (owner < 0) before += red[w];
  }
  if (owner < 0) {
    owner = last_nonempty;
    before = 0.0f;
    for (int w = 0; w < owner; ++w) before += red[w];
  }
  if (wave != owner) return;
  int64_t pick = -1, last_kept = -1;
  float run = before;
  for (int64_t i0 = begin; i0 < end && pick < 0; i0 += 64) {
    const int64_t i = i0 + lane;
    const bool in = i < end && row.key(i) >= thr;
    const float wgt = in ? weight(i) : 0.0f;
    float incl = wgt;                          // inclusive scan over the 64 lanes
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float up = __shfl_up(incl, o);
      if (lane >= o) incl += up;
    }
    const unsigned long long crossed = __builtin_amdgcn_ballot_w64(in && run + incl > target);
    const unsigned long long kept_mask = __builtin_amdgcn_ballot_w64(in);
    if (kept_mask) last_kept = i0 + 63 - __builtin_clzll(kept_mask);
    if (crossed) pick = i0 + __builtin_ctzll(crossed);
    run += __shfl(incl, 63);
  }
  if (pick < 0) pick = last_kept >= 0 ? last_kept : best_i;
  if (lane == 0) out[b] = pick;
}

}  // namespace pa

using namespace pa;

extern "C" int pa_sample(const void* logits, int dtype, int64_t row_stride, int64_t batch, int64_t vocab,
                         float temperature, float top_p, const float* uniforms, int64_t* out, void* stream) {
  if (batch < 0 || vocab <= 0) return fail(PA_ERR_BAD_ARG, "pa_sample: negative or zero size");
  if (batch == 0) return PA_OK;
  if (!logits || !out) return fail(PA_ERR_BAD_ARG, "pa_sample: null pointer");
  if (row_stride < vocab) return fail(PA_ERR_BAD_ARG, "pa_sample: row stride smaller than the vocabulary");
  if (temperature > 0.0f && !uniforms) return fail(PA_ERR_BAD_ARG, "pa_sample: sampling needs one uniform number per row");
  if (!(top_p > 0.0f)) return fail(PA_ERR_BAD_ARG, "pa_sample: top_p must be positive");
  if (batch > 0x7fffffff) return fail(PA_ERR_UNSUPPORTED, "pa_sample: batch too large");
  dim3 grid((unsigned)batch);
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case PA_DTYPE_F16:
      hipLaunchKernelGGL(sample_kernel<PA_DTYPE_F16>, grid, dim3(kSampleThreads), 0, st, logits, row_stride, vocab,
                         temperature, top_p, uniforms, out);
      break;
    case PA_DTYPE_BF16:
      hipLaunchKernelGGL(sample_kernel<PA_DTYPE_BF16>, grid, dim3(kSampleThreads), 0, st, logits, row_stride, vocab,
                         temperature, top_p, uniforms, out);
      break;
    case PA_DTYPE_F32:
      hipLaunchKernelGGL(sample_kernel<PA_DTYPE_F32>, grid, dim3(kSampleThreads), 0, st, logits, row_stride, vocab,
                         temperature, top_p, uniforms, out);
      break;
    default:
      return fail(PA_ERR_UNSUPPORTED, "pa_sample: dtype must be f16, bf16 or f32");
  }
  return check_launch("pa_sample");
}
