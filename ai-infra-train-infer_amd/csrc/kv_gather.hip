// Paged KV cache -> dense per-sequence K / V in head-major layout (gfx950).
//
// The reference's shipped decode mode drives a HuggingFace model: every step it rebuilds that
// model's past_key_values from the paged cache (ModelRunner._load_kv_from_paged_cache,
// src/inference/model_runner.py:340-420).  It computes the slot of every (sequence, position) in
// Python with an .item() per entry, gathers with an index tensor, zeroes the rows past each
// sequence's length and transposes [batch, len, heads, dim] -> [batch, heads, len, dim] with a
// copy, per layer.  All of that is one byte-moving pass: a workgroup takes 16 consecutive positions
// of one sequence (for block_size >= 16 one contiguous piece of a cache block: heads x dim x 16
// tokens), and writes them as `heads` runs of 16 x dim contiguous elements; positions at or past
// the sequence's length are written as zeros.  16-byte accesses, K and V in one launch.
// HBM-bound: every gathered byte is read once and written once.
#include "pa_common.hpp"
#include "pa_host.hpp"

namespace pa {

constexpr int kGatherTokens = 16;     // positions per workgroup

__global__ __launch_bounds__(256) void gather_kv_kernel(const uint8_t* __restrict__ k_cache,
                                                        const uint8_t* __restrict__ v_cache,
                                                        const int32_t* __restrict__ block_tables, int64_t bt_stride,
                                                        const int32_t* __restrict__ context_lens, int len_offset,
                                                        uint8_t* __restrict__ k_out, uint8_t* __restrict__ v_out,
                                                        int num_kv_heads, int row_bytes /* head_dim * element size */,
                                                        int block_size, int num_blocks, int table_width, int out_len) {
  const int b = blockIdx.y;
  const uint8_t* cache = blockIdx.z ? v_cache : k_cache;
  uint8_t* out = blockIdx.z ? v_out : k_out;
  const int pos0 = blockIdx.x * kGatherTokens;
  const int len = max(context_lens[b] - len_offset, 0);        // positions that hold tokens
  const int pieces_per_row = row_bytes >> 4;                     // 16-byte pieces of one (token, head) row
  const int pieces_per_token = pieces_per_row * num_kv_heads;
  const int total = pieces_per_token * kGatherTokens;
  const int64_t token_bytes = (int64_t)num_kv_heads * row_bytes;
  for (int i = threadIdx.x; i < total; i += 256) {
    const int t = i / pieces_per_token;
    const int rem = i - t * pieces_per_token;
    const int h = rem / pieces_per_row;
    const int c = rem - h * pieces_per_row;
    const int pos = pos0 + t;
    if (pos >= out_len) break;                                   // t grows with i
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (pos < len) {
      const int col = pos / block_size;
      const int blk = col < table_width ? block_tables[(int64_t)b * bt_stride + col] : -1;
      if (blk >= 0 && blk < num_blocks) {
        const int64_t slot = (int64_t)blk * block_size + pos % block_size;
        // read once per launch: a streaming (non-temporal) load
        typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
        const u4_t w = __builtin_nontemporal_load((const u4_t*)(cache + slot * token_bytes + (int64_t)h * row_bytes + (c << 4)));
        v = make_uint4(w[0], w[1], w[2], w[3]);
      }
    }
    {
      typedef uint32_t u4s_t __attribute__((ext_vector_type(4)));
      const u4s_t w2 = {v.x, v.y, v.z, v.w};
      __builtin_nontemporal_store(w2, (u4s_t*)(out + (((int64_t)b * num_kv_heads + h) * out_len + pos) * row_bytes + (c << 4)));
    }
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_gather_kv(const void* k_cache, const void* v_cache, const int32_t* block_tables, int64_t bt_stride,
                            int64_t table_width, const int32_t* context_lens, int64_t len_offset, void* k_out,
                            void* v_out, int64_t batch, int64_t num_kv_heads, int64_t head_dim, int64_t elem_bytes,
                            int64_t block_size, int64_t num_blocks, int64_t out_len, void* stream) {
  if (batch < 0 || out_len < 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 || num_blocks <= 0 ||
      table_width < 0 || len_offset < 0)
    return fail(PA_ERR_BAD_ARG, "pa_gather_kv: negative or zero size");
  if (batch == 0 || out_len == 0) return PA_OK;
  if (!k_cache || !v_cache || !block_tables || !context_lens || !k_out || !v_out)
    return fail(PA_ERR_BAD_ARG, "pa_gather_kv: null pointer");
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4)
    return fail(PA_ERR_UNSUPPORTED, "pa_gather_kv: element size must be 1, 2 or 4 bytes");
  const int64_t row_bytes = head_dim * elem_bytes;
  if (row_bytes % 16 != 0) return fail(PA_ERR_UNSUPPORTED, "pa_gather_kv: head_dim x element size must be a multiple of 16 bytes");
  if (!aligned16(k_cache) || !aligned16(v_cache) || !aligned16(k_out) || !aligned16(v_out))
    return fail(PA_ERR_BAD_ARG, "pa_gather_kv: caches and outputs must be 16-byte aligned");
  if (bt_stride < table_width) return fail(PA_ERR_BAD_ARG, "pa_gather_kv: table stride smaller than its width");
  if (batch > 65535 || num_kv_heads > 65535 || row_bytes > (1 << 20) || out_len > INT32_MAX || len_offset > INT32_MAX ||
      num_blocks > INT32_MAX || block_size > INT32_MAX || table_width > INT32_MAX)
    return fail(PA_ERR_UNSUPPORTED, "pa_gather_kv: size too large for one launch");
  const int64_t chunks = (out_len + kGatherTokens - 1) / kGatherTokens;
  if (chunks > INT32_MAX) return fail(PA_ERR_UNSUPPORTED, "pa_gather_kv: out_len too large");
  dim3 grid((unsigned)chunks, (unsigned)batch, 2);
  hipLaunchKernelGGL(gather_kv_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)k_cache,
                     (const uint8_t*)v_cache, block_tables, bt_stride, context_lens, (int)len_offset, (uint8_t*)k_out,
                     (uint8_t*)v_out, (int)num_kv_heads, (int)row_bytes, (int)block_size, (int)num_blocks,
                     (int)table_width, (int)out_len);
  return check_launch("pa_gather_kv");
}
