// Chunked-prefill paged attention (MFMA) — entry point.
#include "pa_common.hpp"
#include "pa_host.hpp"

using namespace pa;

extern "C" int pa_prefill(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
                          const void* v_cache, const float* k_scale, const float* v_scale,
                          int kv_dtype, const int32_t* block_tables, int64_t bt_stride,
                          const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, void* out,
                          int64_t out_token_stride, int64_t num_seqs, int64_t max_seqlen_q,
                          int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                          int64_t block_size, int64_t num_blocks, float scale, void* stream) {
  return fail(PA_ERR_UNSUPPORTED, "pa_prefill: kernel not built in this revision");
}
