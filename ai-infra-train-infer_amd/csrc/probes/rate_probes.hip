// Measuring aids: what the matrix pipe and the memory system sustain.
//
// The chunked-prefill kernel is judged against the dense fp16 MFMA rate of the GPU.  That rate
// depends on the operands: the clocks of the part drop under a loop of matrix instructions, and
// further when the operands toggle.  pa_mfma_rate_probe runs nothing but independent
// v_mfma_f32_32x32x16_f16 on every SIMD of the GPU (8 waves per CU, four accumulator chains per
// wave, operands from registers) on operands the caller supplies - constant ones, or the kind of
// data the attention kernels see - so that a benchmark can put the sustained rate beside the
// nominal one.  pa_hbm_read_probe streams a buffer once with 16-byte loads (ordinary or non-temporal),
// every workgroup its own contiguous chunk, four loads per lane in flight: the plain read rate of the
// GPU, which the decode kernels' achieved bytes per second are put beside.  No counterparts in the reference.
// Part of the measuring library libpa_probes.so (pa_probes.h), not of the product library.
#include "pa_common.hpp"
#include "pa_host.hpp"
#include "pa_probes.h"

namespace pa {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kProbeOperands = 65536;   // fp16 values the caller supplies
constexpr int kProbeProductsPerStep = 16;

__global__ __launch_bounds__(512, 1) void mfma_rate_probe_kernel(const _Float16* src, int64_t steps, float* sink) {
  half8_t a[8], b[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      a[j][i] = src[(threadIdx.x * 64 + j * 8 + i) & (kProbeOperands - 1)];
      b[j][i] = src[(threadIdx.x * 64 + kProbeOperands / 2 + j * 8 + i) & (kProbeOperands - 1)];
    }
  float16_t o[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[j][i] = 0.0f;
  for (int64_t it = 0; it < steps; ++it) {
#pragma unroll
    for (int j = 0; j < kProbeProductsPerStep; ++j)
      o[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j & 7], b[(j + (j >> 3)) & 7], o[j & 3], 0, 0, 0);
  }
  float r = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) r += o[j][0] + o[j][9];
  if (threadIdx.x == 0) sink[blockIdx.x] = r;   // keeps the products alive
}

// Every workgroup reads `per_group` 16-byte words starting at its own offset and leaves the XOR of
// all of them (folded to one word per workgroup) in `sink`.  STREAM: non-temporal loads, as the
// decode kernels read private K/V.
template <bool STREAM>
__global__ __launch_bounds__(256) void hbm_read_probe_kernel(const uint8_t* __restrict__ src, int64_t per_group, uint32_t* sink) {
  typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
  const u4_t* q = (const u4_t*)src + (int64_t)blockIdx.x * per_group;
  auto ld = [&](int64_t i) __attribute__((always_inline)) -> u4_t {
    if constexpr (STREAM) return __builtin_nontemporal_load(q + i);
    else return q[i];
  };
  u4_t acc = {0u, 0u, 0u, 0u};
  int64_t i = threadIdx.x;
  for (; i + 3 * 256 < per_group; i += 4 * 256) {
    const u4_t a = ld(i), b = ld(i + 256), c = ld(i + 512), d = ld(i + 768);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < per_group; i += 256) acc ^= ld(i);
  uint32_t x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) x ^= __shfl_xor(x, off);
  __shared__ uint32_t part[4];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = x;
  __syncthreads();
  if (threadIdx.x == 0) sink[blockIdx.x] = part[0] ^ part[1] ^ part[2] ^ part[3];
}

}  // namespace pa

using namespace pa;

extern "C" int64_t pa_hbm_read_probe(const void* src, int64_t bytes, int64_t groups, int streaming, uint32_t* sink,
                                     int64_t sink_words, void* stream) {
  if (!src || !sink) return fail(PA_ERR_BAD_ARG, "pa_hbm_read_probe: null pointer");
  if (sink_words < groups) return fail(PA_ERR_BAD_ARG, "pa_hbm_read_probe: sink must hold one word per workgroup");
  if (groups <= 0 || groups > 0x7fffffff || bytes <= 0) return fail(PA_ERR_BAD_ARG, "pa_hbm_read_probe: bad size");
  if (!aligned16(src)) return fail(PA_ERR_BAD_ARG, "pa_hbm_read_probe: buffer must be 16-byte aligned");
  const int64_t per_group = bytes / 16 / groups;
  if (per_group <= 0) return fail(PA_ERR_BAD_ARG, "pa_hbm_read_probe: fewer than 16 bytes per workgroup");
  if (streaming)
    hipLaunchKernelGGL(hbm_read_probe_kernel<true>, dim3((unsigned)groups), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t*)src, per_group, sink);
  else
    hipLaunchKernelGGL(hbm_read_probe_kernel<false>, dim3((unsigned)groups), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t*)src, per_group, sink);
  const int rc = check_launch("pa_hbm_read_probe");
  if (rc != PA_OK) return rc;
  return per_group * groups * 16;   // bytes read
}

extern "C" int64_t pa_mfma_rate_probe(const void* operands_f16, int64_t num_operands, int64_t steps, float* sink,
                                      int64_t sink_floats, void* stream) {
  if (!operands_f16 || !sink) return fail(PA_ERR_BAD_ARG, "pa_mfma_rate_probe: null pointer");
  if (steps <= 0 || steps > (int64_t(1) << 24)) return fail(PA_ERR_BAD_ARG, "pa_mfma_rate_probe: steps must be in 1 .. 2^24");
  if (num_operands < kProbeOperands) return fail(PA_ERR_BAD_ARG, "pa_mfma_rate_probe: operands_f16 must hold 65536 values");
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
    return fail(PA_ERR_LAUNCH, "pa_mfma_rate_probe: cannot query the device");
  const int cus = prop.multiProcessorCount;
  if (sink_floats < cus) return fail(PA_ERR_BAD_ARG, "pa_mfma_rate_probe: sink must hold one float per compute unit");
  hipLaunchKernelGGL(mfma_rate_probe_kernel, dim3((unsigned)cus), dim3(512), 0, (hipStream_t)stream,
                     (const _Float16*)operands_f16, steps, sink);
  const int rc = check_launch("pa_mfma_rate_probe");
  if (rc != PA_OK) return rc;
  // floating-point operations of the launch: workgroups x 8 waves x steps x products x 2 * 32 * 32 * 16
  return (int64_t)cus * 8 * steps * kProbeProductsPerStep * 32768;
}
