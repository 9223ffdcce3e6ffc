// Whole-block copies inside the paged KV pool (gfx950): the device half of copy-on-write.
//
// When a sequence appends to a block it shares with another (a forked sample whose prompt ends
// in the middle of a block), the block's contents are first copied to a private block, in every
// layer and for K and V alike.  The reference counts references per block
// (src/inference/kv_cache.py:42-62, 195-212) but never shares one: its K-sample path notes that
// sharing needs exactly this copy (src/inference/engine.py:1108-1113).
//
// The pool tensor is [planes][num_blocks][block_bytes] with planes = 2 x layers for the K/V
// tensor and = layers for each fp8 scale tensor, so one launch moves a block in all planes:
// grid.x walks the block in 16-byte (or 4-byte) pieces, grid.y = plane, grid.z = (src, dst) pair.
// HBM-bound and tiny (a 32 KiB block x 56 planes = 1.8 MB per pair at the Qwen3-0.6B shape).
#include "pa_common.hpp"
#include "pa_host.hpp"

namespace pa {

template <typename T>
__global__ __launch_bounds__(256) void copy_blocks_kernel(uint8_t* __restrict__ pool, int64_t plane_stride_b,
                                                          int64_t block_bytes, int64_t num_blocks,
                                                          const int32_t* __restrict__ pairs) {
  const int64_t src = pairs[2 * blockIdx.z];
  const int64_t dst = pairs[2 * blockIdx.z + 1];
  if (src < 0 || dst < 0 || src >= num_blocks || dst >= num_blocks || src == dst) return;
  uint8_t* plane = pool + (int64_t)blockIdx.y * plane_stride_b;
  const T* s = (const T*)(plane + src * block_bytes);
  T* d = (T*)(plane + dst * block_bytes);
  const int64_t n = block_bytes / (int64_t)sizeof(T);
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) d[i] = s[i];
}

}  // namespace pa

using namespace pa;

extern "C" int pa_copy_blocks(void* pool, int64_t num_planes, int64_t plane_stride_bytes, int64_t block_bytes,
                              int64_t num_blocks, const int32_t* pairs, int64_t num_pairs, void* stream) {
  if (num_planes < 0 || num_pairs < 0 || block_bytes <= 0 || num_blocks <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_copy_blocks: negative or zero size");
  if (num_planes == 0 || num_pairs == 0) return PA_OK;
  if (!pool || !pairs) return fail(PA_ERR_BAD_ARG, "pa_copy_blocks: null pointer");
  if (plane_stride_bytes < num_blocks * block_bytes)
    return fail(PA_ERR_BAD_ARG, "pa_copy_blocks: plane stride smaller than a plane");
  if (block_bytes % 4 != 0 || plane_stride_bytes % 4 != 0 || (reinterpret_cast<uintptr_t>(pool) & 3u) != 0)
    return fail(PA_ERR_UNSUPPORTED, "pa_copy_blocks: sizes and base must be multiples of 4 bytes");
  if (num_planes > 65535 || num_pairs > 65535)
    return fail(PA_ERR_UNSUPPORTED, "pa_copy_blocks: more than 65535 planes or pairs in one launch");
  const bool wide = block_bytes % 16 == 0 && plane_stride_bytes % 16 == 0 && aligned16(pool);
  const int64_t pieces = block_bytes / (wide ? 16 : 4);
  const unsigned gx = (unsigned)((pieces + 255) / 256 < 64 ? (pieces + 255) / 256 : 64);
  dim3 grid(gx, (unsigned)num_planes, (unsigned)num_pairs);
  hipStream_t st = (hipStream_t)stream;
  if (wide)
    hipLaunchKernelGGL(copy_blocks_kernel<uint4>, grid, dim3(256), 0, st, (uint8_t*)pool, plane_stride_bytes,
                       block_bytes, num_blocks, pairs);
  else
    hipLaunchKernelGGL(copy_blocks_kernel<uint32_t>, grid, dim3(256), 0, st, (uint8_t*)pool, plane_stride_bytes,
                       block_bytes, num_blocks, pairs);
  return check_launch("pa_copy_blocks");
}
