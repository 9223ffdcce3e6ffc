// Physical cache slots of tokens, computed on the device (gfx950).
//
// The reference's batched decode derives the slot of every sequence's new token on the host,
// reading position and block id back from the GPU one element at a time
// (src/inference/model_runner.py:670-680: two .item() synchronisations per sequence), and its
// prefill builds the same list in Python loops (model_runner.py:493-511).  Both are
//     slot(token) = block_table[row][position / block_size] * block_size + position % block_size
// over tensors that already sit in HBM, so one small launch does it without leaving the stream:
// one thread per token; the token's table row is its own index (decode) or is found by bisection
// of cu_seqlens_q (prefill chunks).  A position that is negative or beyond the table, and a
// block id outside the pool, give slot -1, which the KV writers skip.
#include "pa_common.hpp"
#include "pa_host.hpp"

namespace pa {

__global__ __launch_bounds__(256) void slot_mapping_kernel(const int64_t* __restrict__ positions,
                                                           const int32_t* __restrict__ cu_seqlens_q,
                                                           const int32_t* __restrict__ block_tables,
                                                           int64_t bt_stride, int32_t* __restrict__ slots,
                                                           int64_t num_tokens, int num_rows, int table_width,
                                                           int block_size, int num_blocks) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= num_tokens) return;
  int row;
  if (cu_seqlens_q) {
    // last row whose first token is <= t; rows without tokens are passed over
    int lo = 0, hi = num_rows;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if ((int64_t)cu_seqlens_q[mid] <= t) lo = mid; else hi = mid;
    }
    row = lo;
    if (t >= (int64_t)cu_seqlens_q[num_rows]) { slots[t] = -1; return; }
  } else {
    row = (int)t;
  }
  const int64_t pos = positions[t];
  int32_t slot = -1;
  if (pos >= 0 && pos / block_size < table_width) {
    const int32_t block = block_tables[(int64_t)row * bt_stride + pos / block_size];
    if (block >= 0 && block < num_blocks) slot = block * block_size + (int32_t)(pos % block_size);
  }
  slots[t] = slot;
}

// Positions and slots of the tokens of a prefill step from its two cumulative length arrays: token t
// belongs to the sequence r whose chunk [cu_q[r], cu_q[r+1]) holds it, the sequence has
// (cu_k[r+1] - cu_k[r]) - (cu_q[r+1] - cu_q[r]) tokens in the cache already, so the token's position
// is that count plus its index in the chunk, and its slot follows from the sequence's table row
// (row_index[r] of the table when given, else r).  One thread per token.
__global__ __launch_bounds__(256) void prefill_metadata_kernel(const int32_t* __restrict__ cu_seqlens_q,
                                                               const int32_t* __restrict__ cu_seqlens_k,
                                                               const int32_t* __restrict__ block_tables,
                                                               int64_t bt_stride, const int32_t* __restrict__ row_index,
                                                               int64_t* __restrict__ positions,
                                                               int32_t* __restrict__ slots, int64_t num_tokens,
                                                               int num_seqs, int table_rows, int table_width,
                                                               int block_size, int num_blocks) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= num_tokens) return;
  if (t >= (int64_t)cu_seqlens_q[num_seqs]) {      // padding behind the last chunk
    positions[t] = 0;
    if (slots) slots[t] = -1;
    return;
  }
  int lo = 0, hi = num_seqs;                       // last sequence whose first token is <= t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)cu_seqlens_q[mid] <= t) lo = mid; else hi = mid;
  }
  const int r = lo;
  const int q0 = cu_seqlens_q[r];
  const int cached = (cu_seqlens_k[r + 1] - cu_seqlens_k[r]) - (cu_seqlens_q[r + 1] - q0);
  const int64_t pos = (int64_t)cached + (t - q0);
  positions[t] = pos;
  if (!slots) return;
  int32_t slot = -1;
  const int row = row_index ? row_index[r] : r;
  if (pos >= 0 && pos / block_size < table_width && row >= 0 && row < table_rows) {
    const int32_t block = block_tables[(int64_t)row * bt_stride + pos / block_size];
    if (block >= 0 && block < num_blocks) slot = block * block_size + (int32_t)(pos % block_size);
  }
  slots[t] = slot;
}

// One decode step of a batch whose metadata lives on the device: every active row (context
// length > 0) gets one token longer, a row whose new token opens a block receives that block's id
// from new_blocks, and position and slot of the new token follow from the row's own table.  One
// thread per row; rows do not interact.
__global__ __launch_bounds__(256) void decode_advance_kernel(int32_t* __restrict__ block_tables, int64_t bt_stride,
                                                             int32_t* __restrict__ context_lens,
                                                             int64_t* __restrict__ positions,
                                                             int32_t* __restrict__ slots,
                                                             const int32_t* __restrict__ new_blocks,
                                                             int64_t* __restrict__ input_ids,
                                                             const int64_t* __restrict__ next_tokens,
                                                             int32_t* __restrict__ fresh, int batch,
                                                             int table_width, int block_size, int num_blocks) {
  const int r = blockIdx.x * 256 + threadIdx.x;
  if (r >= batch) return;
  const int len = context_lens[r];
  if (len <= 0) {            // inactive row: writes nothing, reads nothing
    slots[r] = -1;
    positions[r] = 0;
    return;
  }
  // the token to feed: what the last step produced for this row, unless the row has just been
  // admitted and still holds the token its prefill produced
  if (fresh && fresh[r]) fresh[r] = 0;
  else if (next_tokens && input_ids) input_ids[r] = next_tokens[r];
  const int pos = len;       // index of the token being written; the context then counts it
  const int col = pos / block_size;
  int32_t block = -1;
  if (col < table_width) {
    int32_t* entry = block_tables + (int64_t)r * bt_stride + col;
    if (new_blocks && new_blocks[r] >= 0) *entry = new_blocks[r];
    block = *entry;
  }
  context_lens[r] = len + 1;
  positions[r] = pos;
  slots[r] = (block >= 0 && block < num_blocks) ? block * block_size + pos % block_size : -1;
}

}  // namespace pa

using namespace pa;

extern "C" int pa_slot_mapping(const int64_t* positions, const int32_t* cu_seqlens_q, const int32_t* block_tables,
                               int64_t bt_stride, int32_t* slots, int64_t num_tokens, int64_t num_rows,
                               int64_t table_width, int64_t block_size, int64_t num_blocks, void* stream) {
  if (num_tokens < 0 || num_rows < 0 || table_width < 0 || block_size <= 0 || num_blocks <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_slot_mapping: negative or zero size");
  if (num_tokens == 0) return PA_OK;
  if (!positions || !block_tables || !slots) return fail(PA_ERR_BAD_ARG, "pa_slot_mapping: null pointer");
  if (num_rows == 0) return fail(PA_ERR_BAD_ARG, "pa_slot_mapping: tokens but no table rows");
  if (!cu_seqlens_q && num_tokens != num_rows)
    return fail(PA_ERR_BAD_ARG, "pa_slot_mapping: without cu_seqlens_q every table row has exactly one token");
  if (bt_stride < table_width) return fail(PA_ERR_BAD_ARG, "pa_slot_mapping: table stride smaller than its width");
  if (num_rows > INT32_MAX || table_width > INT32_MAX || num_blocks * block_size > INT32_MAX)
    return fail(PA_ERR_UNSUPPORTED, "pa_slot_mapping: slots must fit int32");
  const int64_t wgs = (num_tokens + 255) / 256;
  if (wgs > INT32_MAX) return fail(PA_ERR_UNSUPPORTED, "pa_slot_mapping: too many tokens for one launch");
  hipLaunchKernelGGL(slot_mapping_kernel, dim3((unsigned)wgs), dim3(256), 0, (hipStream_t)stream, positions,
                     cu_seqlens_q, block_tables, bt_stride, slots, num_tokens, (int)num_rows, (int)table_width,
                     (int)block_size, (int)num_blocks);
  return check_launch("pa_slot_mapping");
}

extern "C" int pa_prefill_metadata(const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* block_tables,
                                   int64_t bt_stride, const int32_t* row_index, int64_t* positions, int32_t* slots,
                                   int64_t num_tokens, int64_t num_seqs, int64_t table_rows, int64_t table_width,
                                   int64_t block_size, int64_t num_blocks, void* stream) {
  if (num_tokens < 0 || num_seqs < 0 || table_rows < 0 || table_width < 0 || block_size <= 0 || num_blocks <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_prefill_metadata: negative or zero size");
  if (num_tokens == 0) return PA_OK;
  if (!cu_seqlens_q || !cu_seqlens_k || !positions) return fail(PA_ERR_BAD_ARG, "pa_prefill_metadata: null pointer");
  if (num_seqs == 0) return fail(PA_ERR_BAD_ARG, "pa_prefill_metadata: tokens but no sequences");
  if (slots && !block_tables) return fail(PA_ERR_BAD_ARG, "pa_prefill_metadata: slots need block tables");
  if (slots && bt_stride < table_width) return fail(PA_ERR_BAD_ARG, "pa_prefill_metadata: table stride smaller than its width");
  if (num_seqs > INT32_MAX || table_rows > INT32_MAX || table_width > INT32_MAX || num_blocks * block_size > INT32_MAX)
    return fail(PA_ERR_UNSUPPORTED, "pa_prefill_metadata: slots must fit int32");
  const int64_t wgs = (num_tokens + 255) / 256;
  if (wgs > INT32_MAX) return fail(PA_ERR_UNSUPPORTED, "pa_prefill_metadata: too many tokens for one launch");
  hipLaunchKernelGGL(prefill_metadata_kernel, dim3((unsigned)wgs), dim3(256), 0, (hipStream_t)stream, cu_seqlens_q,
                     cu_seqlens_k, block_tables, bt_stride, row_index, positions, slots, num_tokens, (int)num_seqs,
                     (int)table_rows, (int)table_width, (int)block_size, (int)num_blocks);
  return check_launch("pa_prefill_metadata");
}

extern "C" int pa_decode_advance(int32_t* block_tables, int64_t bt_stride, int32_t* context_lens, int64_t* positions,
                                 int32_t* slots, const int32_t* new_blocks, int64_t* input_ids,
                                 const int64_t* next_tokens, int32_t* fresh, int64_t batch, int64_t table_width,
                                 int64_t block_size, int64_t num_blocks, void* stream) {
  if (batch < 0 || table_width < 0 || block_size <= 0 || num_blocks <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_decode_advance: negative or zero size");
  if (batch == 0) return PA_OK;
  if (!block_tables || !context_lens || !positions || !slots)
    return fail(PA_ERR_BAD_ARG, "pa_decode_advance: null pointer");
  if (next_tokens && !input_ids) return fail(PA_ERR_BAD_ARG, "pa_decode_advance: next_tokens without input_ids");
  if (bt_stride < table_width) return fail(PA_ERR_BAD_ARG, "pa_decode_advance: table stride smaller than its width");
  if (batch > INT32_MAX || table_width > INT32_MAX || num_blocks * block_size > INT32_MAX)
    return fail(PA_ERR_UNSUPPORTED, "pa_decode_advance: slots must fit int32");
  hipLaunchKernelGGL(decode_advance_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     block_tables, bt_stride, context_lens, positions, slots, new_blocks, input_ids, next_tokens,
                     fresh, (int)batch, (int)table_width, (int)block_size, (int)num_blocks);
  return check_launch("pa_decode_advance");
}
