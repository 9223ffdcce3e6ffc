// The element-wise steps of a Qwen3 decoder block around its GEMMs and attention (gfx950):
//
//   pa_add_rms_norm   h = h + delta (a block's residual add, src/distributed/tensor_parallel.py:640-651)
//                     followed by the next RMSNorm (tensor_parallel.py:78-84:
//                     y = w * (x * rsqrt(mean(x^2) + eps)) in fp32, cast back), one launch
//   pa_silu_mul       silu(gate) * up of the SwiGLU MLP (tensor_parallel.py:295-299)
//
// As torch ops a norm is seven launches (cast, square, mean, add, rsqrt, two multiplies, cast) and
// the residual add and the activation three more; a decode step has 64 rows, so each launch is
// pure latency and a 28-layer step spends more time in them than in attention.  Here one wave
// owns one row: 16-byte accesses, every load of the row in flight before any arithmetic, the
// sum of squares reduced across the wave, and the row never leaves registers between the add,
// the norm and the two stores.  Roundings are those of the separate ops: the residual sum is
// rounded to the activation dtype before it is normalised (and is what the next block adds to),
// the norm multiplies x by the reciprocal root first and by the weight second, both in fp32,
// and rounds once; silu is rounded to the activation dtype before the product, as F.silu(gate)
// * up does.
#include "pa_common.hpp"
#include "pa_host.hpp"

namespace pa {

constexpr int kRowsPerGroup = 4;      // waves (= rows) per workgroup

template <int DT>
__device__ __forceinline__ void load8(const void* p, int64_t i, float (&x)[8]) {
  load8_as_f32(p, i, DT, x);
}

template <int DT>
__device__ __forceinline__ float round_dt(float x) {
  if constexpr (DT == PA_DTYPE_F16) return f16_bits_to_f32(f32_to_f16_bits(x));
  else if constexpr (DT == PA_DTYPE_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(x));
  else return x;
}

template <int DT>
__device__ __forceinline__ void store8(void* p, int64_t i, const float (&x)[8]) {
  if constexpr (DT == PA_DTYPE_F32) {
    *(float4*)((float*)p + i) = make_float4(x[0], x[1], x[2], x[3]);
    *(float4*)((float*)p + i + 4) = make_float4(x[4], x[5], x[6], x[7]);
  } else {
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t lo = DT == PA_DTYPE_F16 ? f32_to_f16_bits(x[2 * k]) : f32_to_bf16_bits(x[2 * k]);
      const uint32_t hi = DT == PA_DTYPE_F16 ? f32_to_f16_bits(x[2 * k + 1]) : f32_to_bf16_bits(x[2 * k + 1]);
      w[k] = lo | (hi << 16);
    }
    *(uint4*)((uint16_t*)p + i) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

struct AddNormParams {
  const void* x;          // [rows, hidden]
  const void* delta;      // optional: added to x first
  const void* weight;     // [hidden]
  void* sum_out;          // optional: x + delta (may be x itself)
  void* normed_out;
  int64_t x_stride, delta_stride, sum_stride, normed_stride;   // elements
  int64_t rows;
  int hidden;
  int weight_dtype;
  float eps;
};

// CH = 8-element chunks a lane holds: the row has at most 64 * CH of them.  Short rows (CH <= 4)
// also keep their delta and weight chunks in registers, so that every load of the row is in
// flight at once; long rows stream those two through as they are used.
template <int DT, int CH>
__global__ __launch_bounds__(64 * kRowsPerGroup) void add_rms_norm_kernel(const AddNormParams p) {
  constexpr bool HOLD = CH <= 4;
  constexpr int HC = HOLD ? CH : 1;
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * kRowsPerGroup + (threadIdx.x >> 6);
  if (r >= p.rows) return;                         // the whole wave
  const int chunks = p.hidden >> 3;
  float x[CH][8], d[HC][8], w[HC][8];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = lane + 64 * j;
#pragma unroll
    for (int e = 0; e < 8; ++e) x[j][e] = 0.0f;
    if (c < chunks) load8<DT>(p.x, r * p.x_stride + c * 8, x[j]);
    if constexpr (HOLD) {
#pragma unroll
      for (int e = 0; e < 8; ++e) d[j][e] = w[j][e] = 0.0f;
      if (c < chunks) {
        if (p.delta) load8<DT>(p.delta, r * p.delta_stride + c * 8, d[j]);
        load8_as_f32(p.weight, c * 8, p.weight_dtype, w[j]);
      }
    }
  }
  float ss = 0.0f;
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = lane + 64 * j;
    if (p.delta) {
      if constexpr (!HOLD) {
#pragma unroll
        for (int e = 0; e < 8; ++e) d[0][e] = 0.0f;
        if (c < chunks) load8<DT>(p.delta, r * p.delta_stride + c * 8, d[0]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) x[j][e] = round_dt<DT>(x[j][e] + d[HOLD ? j : 0][e]);
      if (p.sum_out && c < chunks) store8<DT>(p.sum_out, r * p.sum_stride + c * 8, x[j]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += x[j][e] * x[j][e];
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
  const float inv = rsqrtf(ss / (float)p.hidden + p.eps);
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = lane + 64 * j;
    if (c < chunks) {
      if constexpr (!HOLD) load8_as_f32(p.weight, c * 8, p.weight_dtype, w[0]);
      float y[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = w[HOLD ? j : 0][e] * (x[j][e] * inv);
      store8<DT>(p.normed_out, r * p.normed_stride + c * 8, y);
    }
  }
}

// out[r, i] = round(silu(gate[r, i])) * up[r, i]; one thread per 8 elements.
template <int DT>
__global__ __launch_bounds__(256) void silu_mul_kernel(const void* __restrict__ gate, const void* __restrict__ up,
                                                       void* __restrict__ out, int64_t gate_stride,
                                                       int64_t up_stride, int64_t out_stride, int64_t rows,
                                                       int chunks_per_row) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * chunks_per_row) return;
  const int64_t r = i / chunks_per_row;
  const int c = (int)(i % chunks_per_row);
  float g[8], u[8];
  load8<DT>(gate, r * gate_stride + c * 8, g);
  load8<DT>(up, r * up_stride + c * 8, u);
#pragma unroll
  for (int e = 0; e < 8; ++e) g[e] = round_dt<DT>(g[e] / (1.0f + __expf(-g[e]))) * u[e];
  store8<DT>(out, r * out_stride + c * 8, g);
}

template <int DT>
int launch_add_rms_norm(const AddNormParams& p, hipStream_t st) {
  const int chunks = p.hidden / 8;
  const dim3 grid((unsigned)((p.rows + kRowsPerGroup - 1) / kRowsPerGroup)), block(64 * kRowsPerGroup);
  if (chunks <= 64 * 2) hipLaunchKernelGGL((add_rms_norm_kernel<DT, 2>), grid, block, 0, st, p);
  else if (chunks <= 64 * 4) hipLaunchKernelGGL((add_rms_norm_kernel<DT, 4>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((add_rms_norm_kernel<DT, 16>), grid, block, 0, st, p);
  return check_launch("pa_add_rms_norm");
}

}  // namespace pa

using namespace pa;

static bool rows16(const void* p, int64_t stride_elems, int64_t elem) {
  return aligned16(p) && (stride_elems * elem) % 16 == 0;
}

extern "C" int pa_add_rms_norm(const void* x, int64_t x_stride, const void* delta, int64_t delta_stride,
                               const void* weight, int weight_dtype, float eps, void* sum_out, int64_t sum_stride,
                               void* normed_out, int64_t normed_stride, int dtype, int64_t rows, int64_t hidden,
                               void* stream) {
  if (rows < 0 || hidden <= 0) return fail(PA_ERR_BAD_ARG, "pa_add_rms_norm: negative or zero size");
  if (rows == 0) return PA_OK;
  if (!x || !weight || !normed_out) return fail(PA_ERR_BAD_ARG, "pa_add_rms_norm: null pointer");
  if (dtype != PA_DTYPE_F16 && dtype != PA_DTYPE_BF16 && dtype != PA_DTYPE_F32)
    return fail(PA_ERR_UNSUPPORTED, "pa_add_rms_norm: dtype must be f16, bf16 or f32");
  if (weight_dtype != PA_DTYPE_F16 && weight_dtype != PA_DTYPE_BF16 && weight_dtype != PA_DTYPE_F32)
    return fail(PA_ERR_UNSUPPORTED, "pa_add_rms_norm: weight dtype must be f16, bf16 or f32");
  if (hidden % 8 != 0 || hidden > 8 * 64 * 16)
    return fail(PA_ERR_UNSUPPORTED, "pa_add_rms_norm: hidden must be a multiple of 8, at most 8192");
  if (!(eps >= 0.0f)) return fail(PA_ERR_BAD_ARG, "pa_add_rms_norm: eps must be non-negative");
  if (sum_out && !delta) return fail(PA_ERR_BAD_ARG, "pa_add_rms_norm: sum_out without delta");
  const int64_t es = dtype == PA_DTYPE_F32 ? 4 : 2;
  const int64_t ws = weight_dtype == PA_DTYPE_F32 ? 4 : 2;
  if (x_stride < hidden || normed_stride < hidden || (delta && delta_stride < hidden) ||
      (sum_out && sum_stride < hidden))
    return fail(PA_ERR_BAD_ARG, "pa_add_rms_norm: row stride smaller than hidden");
  if (!rows16(x, x_stride, es) || !rows16(normed_out, normed_stride, es) || !rows16(weight, 8, ws) ||
      (delta && !rows16(delta, delta_stride, es)) || (sum_out && !rows16(sum_out, sum_stride, es)))
    return fail(PA_ERR_UNSUPPORTED, "pa_add_rms_norm: rows and weight must be 16-byte aligned");
  AddNormParams p;
  p.x = x; p.delta = delta; p.weight = weight; p.sum_out = sum_out; p.normed_out = normed_out;
  p.x_stride = x_stride; p.delta_stride = delta_stride; p.sum_stride = sum_stride; p.normed_stride = normed_stride;
  p.rows = rows; p.hidden = (int)hidden; p.weight_dtype = weight_dtype; p.eps = eps;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == PA_DTYPE_F16) return launch_add_rms_norm<PA_DTYPE_F16>(p, st);
  if (dtype == PA_DTYPE_BF16) return launch_add_rms_norm<PA_DTYPE_BF16>(p, st);
  return launch_add_rms_norm<PA_DTYPE_F32>(p, st);
}

extern "C" int pa_silu_mul(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride, void* out,
                           int64_t out_stride, int dtype, int64_t rows, int64_t width, void* stream) {
  if (rows < 0 || width <= 0) return fail(PA_ERR_BAD_ARG, "pa_silu_mul: negative or zero size");
  if (rows == 0) return PA_OK;
  if (!gate || !up || !out) return fail(PA_ERR_BAD_ARG, "pa_silu_mul: null pointer");
  if (dtype != PA_DTYPE_F16 && dtype != PA_DTYPE_BF16 && dtype != PA_DTYPE_F32)
    return fail(PA_ERR_UNSUPPORTED, "pa_silu_mul: dtype must be f16, bf16 or f32");
  if (width % 8 != 0) return fail(PA_ERR_UNSUPPORTED, "pa_silu_mul: width must be a multiple of 8");
  if (gate_stride < width || up_stride < width || out_stride < width)
    return fail(PA_ERR_BAD_ARG, "pa_silu_mul: row stride smaller than width");
  const int64_t es = dtype == PA_DTYPE_F32 ? 4 : 2;
  if (!rows16(gate, gate_stride, es) || !rows16(up, up_stride, es) || !rows16(out, out_stride, es))
    return fail(PA_ERR_UNSUPPORTED, "pa_silu_mul: rows must be 16-byte aligned");
  const int64_t chunks = width / 8;
  const int64_t wgs = (rows * chunks + 255) / 256;
  if (wgs > INT32_MAX || chunks > INT32_MAX) return fail(PA_ERR_UNSUPPORTED, "pa_silu_mul: too large for one launch");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)wgs), block(256);
  if (dtype == PA_DTYPE_F16)
    hipLaunchKernelGGL(silu_mul_kernel<PA_DTYPE_F16>, grid, block, 0, st, gate, up, out, gate_stride, up_stride,
                       out_stride, rows, (int)chunks);
  else if (dtype == PA_DTYPE_BF16)
    hipLaunchKernelGGL(silu_mul_kernel<PA_DTYPE_BF16>, grid, block, 0, st, gate, up, out, gate_stride, up_stride,
                       out_stride, rows, (int)chunks);
  else
    hipLaunchKernelGGL(silu_mul_kernel<PA_DTYPE_F32>, grid, block, 0, st, gate, up, out, gate_stride, up_stride,
                       out_stride, rows, (int)chunks);
  return check_launch("pa_silu_mul");
}
