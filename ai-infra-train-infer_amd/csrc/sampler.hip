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
// {j : l_j >= t*} with t* the smallest logit whose G is <= top_p: t* is found four bits at a time over
// the ordered bit patterns of the logit type (4 passes for fp16 / bf16 rows, 8 for fp32), each pass
// sorting the weights of the still-undecided logits into 16 buckets, with the row resident in L2.  The draw itself is an inverse-CDF lookup in index order with a uniform
// number supplied by the caller, so a step is reproducible and needs no generator state on the
// device: the first index j with sum_{i <= j, kept} p_i > u * (kept mass).
// Logits tied with t* all stay (a sort keeps an implementation-defined subset of such a tie).
#include "pa_common.hpp"
#include "pa_host.hpp"

#include <math.h>

namespace pa {

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / 64;
constexpr int kMaxChunks = 64;                 // chunks of a wave's range whose sums are listed in LDS
constexpr int kBuckets = 16;                   // key bits per pass of the threshold search: 4
static_assert(kBuckets == kSampleWaves, "one wave adds up one bucket");

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
    // four 16-byte pieces per thread in flight: with one, a pass over the row is a chain of
    // L2 latencies (19 of them for a 152k-entry fp16 row)
    constexpr int UNROLL = 4;
    auto apply = [&](int64_t c, const uint4& w) __attribute__((always_inline)) {
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
    };
    int64_t c = threadIdx.x;
    for (; c + (UNROLL - 1) * kSampleThreads < nvec; c += UNROLL * kSampleThreads) {
      uint4 w[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) w[u] = ((const uint4*)p)[c + u * kSampleThreads];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) apply(c + u * kSampleThreads, w[u]);
    }
    for (; c < nvec; c += kSampleThreads) apply(c, ((const uint4*)p)[c]);
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
  __shared__ float hist[kBuckets][kSampleThreads];     // a thread's own 16 slots: column tid
  __shared__ float chunk[kSampleWaves][kMaxChunks];    // kept weight per chunk of a wave's range
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
  // the threshold search weighs with the hardware exponential (results below 2^-126 flush to
  // zero, far beneath anything that can move a cut)
  auto fast_weight = [&](uint32_t bits) { return __builtin_amdgcn_exp2f((Row<DT>::bits_value(bits) - best) * c); };

  // ---- nucleus threshold: smallest key t with mass(key > t) <= top_p * Z ---------------------------
  // Four key bits per pass.  A pass sorts the weights of the keys that share the bits found so
  // far into 16 buckets by their next four bits; every thread adds into its own 16 LDS slots, so
  // there is no atomic traffic and the sums do not depend on timing.  The bucket in which the
  // mass above crosses top_p * Z fixes the next four bits.  The first pass weighs every entry
  // (its buckets also add up to Z); later passes only those inside one bucket of the one before.
  uint32_t thr = 0;            // keep everything
  if (top_p < 1.0f) {
    constexpr int BITS = DT == PA_DTYPE_F32 ? 32 : 16;
    float above = 0.0f;        // mass of the keys above the prefix found so far
    float limit = 0.0f;
    uint32_t prefix = 0;
    for (int shift = BITS - 4; shift >= 0; shift -= 4) {
#pragma unroll
      for (int j = 0; j < kBuckets; ++j) hist[j][tid] = 0.0f;
      const bool first = shift == BITS - 4;
      // The keys that share `prefix` are the raw bit patterns that share raw_prefix (the key
      // transform flips all bits of a negative number and the sign bit of the others), so the
      // test that nearly every entry fails costs a shift and a compare.
      const int n = BITS - 4 - shift;                    // bits in prefix
      const uint32_t ones = n ? (0xffffffffu >> (32 - n)) : 0u;
      const uint32_t raw_prefix = (n && !((prefix >> (n - 1)) & 1u)) ? (~prefix & ones) : (prefix ^ (n ? 1u << (n - 1) : 0u));
      row.for_each(vocab, [&](int64_t, uint32_t bits) {
        if (first || (bits >> (shift + 4)) == raw_prefix) {
          const uint32_t k = Row<DT>::bits_key(bits);
          hist[(k >> shift) & (kBuckets - 1)][tid] += fast_weight(bits);
        }
      });
      __syncthreads();
      // wave w adds up bucket w: 16 slots per lane, then across the lanes, always in the same order
      {
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < kSampleThreads / 64; ++j) sum += hist[wave][lane + 64 * j];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
        if (lane == 0) red[wave] = sum;
      }
      __syncthreads();
      float m[kBuckets];
#pragma unroll
      for (int j = 0; j < kBuckets; ++j) m[j] = red[j];
      if (first) {
        float z = 0.0f;
#pragma unroll
        for (int j = 0; j < kBuckets; ++j) z += m[j];
        limit = top_p * z;
      }
      // smallest bucket whose mass-above is within the limit (the top bucket's always is)
      int pick = kBuckets - 1;
      float run = above, above_pick = above;
#pragma unroll
      for (int j = kBuckets - 1; j > 0; --j) {
        run += m[j];                       // mass above bucket j - 1
        if (run <= limit) { pick = j - 1; above_pick = run; }
      }
      above = above_pick;
      prefix = (prefix << 4) | (uint32_t)pick;
      __syncthreads();                     // red and hist are reused by the next pass
    }
    thr = prefix;
  }

  // ---- inverse CDF in index order over the kept tokens -----------------------------------------------
  // Wave w owns the contiguous range [w * span, (w + 1) * span); a lane takes PER consecutive
  // entries (one 16-byte load) per step, so lane order is index order.
  constexpr int PER = DT == PA_DTYPE_F32 ? 4 : 8;
  constexpr int ES = DT == PA_DTYPE_F32 ? 4 : 2;
  const int64_t span = ((vocab + kSampleWaves - 1) / kSampleWaves + 64 * PER - 1) / (64 * PER) * (64 * PER);
  const int64_t begin = (int64_t)wave * span, end = begin + span < vocab ? begin + span : vocab;
  const bool wide = (reinterpret_cast<uintptr_t>(row.p) & 15u) == 0;
  // the kept weights of the PER entries starting at i0 (zero outside the range or below the cut)
  auto piece = [&](int64_t i0, float (&wgt)[PER], bool (&in)[PER]) __attribute__((always_inline)) {
    uint32_t bits[PER];
    if (wide && i0 + PER <= end) {
      const uint4 w = *(const uint4*)((const uint8_t*)row.p + i0 * ES);
      const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if constexpr (DT == PA_DTYPE_F32) bits[k] = ww[k];
        else { bits[2 * k] = ww[k] & 0xffffu; bits[2 * k + 1] = ww[k] >> 16; }
      }
#pragma unroll
      for (int e = 0; e < PER; ++e) in[e] = true;
    } else {
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        in[e] = i0 + e < end;
        bits[e] = 0;
        if (in[e]) {
          if constexpr (DT == PA_DTYPE_F32) bits[e] = __float_as_uint(((const float*)row.p)[i0 + e]);
          else bits[e] = ((const uint16_t*)row.p)[i0 + e];
        }
      }
    }
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      in[e] = in[e] && Row<DT>::bits_key(bits[e]) >= thr;
      wgt[e] = in[e] ? fast_weight(bits[e]) : 0.0f;
    }
  };
  // pass 1, all waves: the kept weight of every 64 * PER-entry chunk of the wave's range, and
  // their sum in chunk order (the owner below re-adds them in the same order)
  const int nchunks = (int)((end > begin ? end - begin + 64 * PER - 1 : 0) / (64 * PER));
  const bool listed = nchunks <= kMaxChunks;       // else: the owner walks its range chunk by chunk
  float mine = 0.0f;
  for (int it = 0; it < nchunks; ++it) {
    float wgt[PER];
    bool in[PER];
    piece(begin + (int64_t)it * 64 * PER + lane * PER, wgt, in);
    float part = 0.0f;
#pragma unroll
    for (int e = 0; e < PER; ++e) part += wgt[e];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o);
    if (listed && lane == 0) chunk[wave][it] = part;
    mine += part;
  }
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
  // pass 2, the owner: the chunk in which the sum passes the target (from the list, else by
  // walking), then the entry inside it
  int64_t pick = -1, last_kept = -1;
  float run = before;
  int first_chunk = 0, last_chunk = nchunks - 1;
  if (listed) {
    int cross = -1, last_nz = -1;
    float r = before;
    for (int it = 0; it < nchunks; ++it) {
      const float cs = chunk[wave][it];
      if (cs > 0.0f) last_nz = it;
      if (cross < 0) { if (r + cs > target) cross = it; else r += cs; }
    }
    if (cross >= 0) { first_chunk = last_chunk = cross; run = r; }
    else { first_chunk = last_chunk = last_nz < 0 ? 0 : last_nz; run = -INFINITY; }   // rounding: take the last kept entry
  }
  for (int it = first_chunk; it <= last_chunk && pick < 0; ++it) {
    const int64_t base = begin + (int64_t)it * 64 * PER;
    float wgt[PER];
    bool in[PER];
    piece(base + lane * PER, wgt, in);
    float lane_sum = 0.0f;
    bool any = false;
#pragma unroll
    for (int e = 0; e < PER; ++e) { lane_sum += wgt[e]; any = any || in[e]; }
    float incl = lane_sum;                     // inclusive scan of the lane totals
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float up = __shfl_up(incl, o);
      if (lane >= o) incl += up;
    }
    const unsigned long long crossed = __builtin_amdgcn_ballot_w64(any && run + incl > target);
    const unsigned long long kept_mask = __builtin_amdgcn_ballot_w64(any);
    if (kept_mask) {                           // last kept entry so far: inside the highest such lane
      const int hl = 63 - __builtin_clzll(kept_mask);
      int last_e = 0;
#pragma unroll
      for (int e = 0; e < PER; ++e) if (in[e]) last_e = e;
      last_kept = base + hl * PER + __shfl(last_e, hl);
    }
    if (crossed) {                             // the first lane whose running sum passes the target
      const int cl = __builtin_ctzll(crossed);
      float acc = run + incl - lane_sum;       // sum before this lane's entries
      int first_e = -1, tail_e = 0;
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        acc += wgt[e];
        if (in[e]) { tail_e = e; if (first_e < 0 && acc > target) first_e = e; }
      }
      if (first_e < 0) first_e = tail_e;       // rounding: the lane total passed, no prefix did
      pick = base + cl * PER + __shfl(first_e, cl);
    }
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
