// Measuring aid: what the matrix pipe sustains.
//
// The chunked-prefill kernel is judged against the dense fp16 MFMA rate of the GPU.  That rate
// depends on the operands: the clocks of the part drop under a loop of matrix instructions, and
// further when the operands toggle.  pa_mfma_rate_probe runs nothing but independent
// v_mfma_f32_32x32x16_f16 on every SIMD of the GPU (8 waves per CU, four accumulator chains per
// wave, operands from registers) on operands the caller supplies - constant ones, or the kind of
// data the attention kernels see - so that a benchmark can put the sustained rate beside the
// nominal one.  No counterpart in the reference.
#include "pa_common.hpp"
#include "pa_host.hpp"

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

}  // namespace pa

using namespace pa;

extern "C" int64_t pa_mfma_rate_probe(const void* operands_f16, int64_t steps, float* sink, void* stream) {
  if (!operands_f16 || !sink) return fail(PA_ERR_BAD_ARG, "pa_mfma_rate_probe: null pointer");
  if (steps <= 0 || steps > (int64_t(1) << 24)) return fail(PA_ERR_BAD_ARG, "pa_mfma_rate_probe: steps must be in 1 .. 2^24");
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
    return fail(PA_ERR_LAUNCH, "pa_mfma_rate_probe: cannot query the device");
  const int cus = prop.multiProcessorCount;
  hipLaunchKernelGGL(mfma_rate_probe_kernel, dim3((unsigned)cus), dim3(512), 0, (hipStream_t)stream,
                     (const _Float16*)operands_f16, steps, sink);
  const int rc = check_launch("pa_mfma_rate_probe");
  if (rc != PA_OK) return rc;
  // floating-point operations of the launch: workgroups x 8 waves x steps x products x 2 * 32 * 32 * 16
  return (int64_t)cus * 8 * steps * kProbeProductsPerStep * 32768;
}
