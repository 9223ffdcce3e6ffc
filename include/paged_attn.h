/*
 * paged_attn.h — C ABI of the MI355X (gfx950) paged-attention library.
 *
 * Every entry point takes raw device pointers, plain integer sizes and a HIP
 * stream handle (void*, a hipStream_t; NULL = the default stream).  Nothing
 * here allocates or frees device memory, synchronises with the host, or keeps
 * a pointer after returning: the caller owns every buffer.  All launches are
 * asynchronous on `stream` and may be recorded into a HIP graph.
 *
 * Return value: PA_OK (0) or a negative PA_ERR_* code; pa_last_error() then
 * holds a message for the calling thread.
 *
 * Data layout (the reference engine's, kept as is):
 *   K or V cache of one layer  [num_blocks, block_size, num_kv_heads, head_dim]
 *                              contiguous, fp16 / bf16 / fp8-e4m3fn
 *                              (reference: src/inference/kv_cache.py:131-174,
 *                               bound per layer at src/inference/model_runner.py:102-116)
 *   k_scale / v_scale          [num_blocks, block_size] fp32, one multiplier per token
 *                              (448 / amax; dequant = fp8 / scale)
 *   slot_mapping               [num_tokens] int32, slot = block_id*block_size + offset,
 *                              negative = skip (src/inference/attention.py:94,132,155)
 *   block_tables               [batch, bt_stride] int32, entries past
 *                              ceil(context_len/block_size) are never dereferenced
 *   context_lens               [batch] int32, 0 = padded row (output row is zeroed)
 */
#ifndef PAGED_ATTN_H_
#define PAGED_ATTN_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PA_OK 0
#define PA_ERR_BAD_ARG (-1)      /* null pointer, negative size, misaligned buffer */
#define PA_ERR_UNSUPPORTED (-2)  /* shape or dtype the kernels are not built for */
#define PA_ERR_LAUNCH (-3)       /* hipGetLastError() reported a failure */
#define PA_ERR_WORKSPACE (-4)    /* workspace missing or too small */

/* element types */
#define PA_DTYPE_F16 0
#define PA_DTYPE_BF16 1
#define PA_DTYPE_F32 2
#define PA_DTYPE_FP8_E4M3 3 /* OCP e4m3fn, the layout of torch.float8_e4m3fn */

/* Library ABI version (bumped when a signature changes); 3 = listed group rows in pa_decode_shared_prefix. */
int pa_version(void);

/* Message for the last non-zero return code on this thread ("" if none). */
const char* pa_last_error(void);

/*
 * Paged KV-cache write, same-dtype bit copy.
 * Replaces: store_kv_cache -> _store_kv_cache_pytorch / _store_kv_cache_triton
 *           (src/inference/attention.py:44-72, 119-135, 141-183).
 * For every token t with 0 <= slot_mapping[t] < total_slots the row
 * key[t, :row_elems] is copied to k_cache[slot, :row_elems] (same for value).
 * Negative slots are skipped; slots >= total_slots are skipped too (the
 * reference would raise an index error on the host).
 *   key/value            [num_tokens, row_elems], token stride given in elements
 *   row_elems            num_kv_heads * head_dim; row_elems*elem_bytes % 16 == 0
 *   elem_bytes           1, 2 or 4
 */
int pa_kv_store(const void* key, const void* value, int64_t key_token_stride,
                int64_t value_token_stride, void* k_cache, void* v_cache,
                const int32_t* slot_mapping, int64_t num_tokens, int64_t row_elems,
                int elem_bytes, int64_t total_slots, void* stream);

/*
 * Paged KV-cache write with per-token FP8-e4m3fn quantisation.
 * Replaces: store_kv_cache -> _store_kv_cache_fp8 (src/inference/attention.py:75-116).
 * Per token and per tensor: amax = max |fp32(x)| over the row, clamped to >= 1e-5;
 * s = fl(fl(1/amax) * 448) in fp32 (how torch evaluates the reference's `448.0 / amax`:
 * reciprocal, then multiply, each correctly rounded); byte = e4m3fn(fp32(x) * s) with
 * round-to-nearest-even and no saturation; bytes go to the cache row, s to
 * the scale slot.  Bytes and scales are bit-identical to the reference arithmetic.
 *   in_dtype             PA_DTYPE_F16 / BF16 / F32
 *   row_elems            num_kv_heads * head_dim, a multiple of 16
 */
int pa_kv_store_fp8(const void* key, const void* value, int in_dtype,
                    int64_t key_token_stride, int64_t value_token_stride, void* k_cache,
                    void* v_cache, float* k_scale, float* v_scale,
                    const int32_t* slot_mapping, int64_t num_tokens, int64_t row_elems,
                    int64_t total_slots, void* stream);

/*
 * Bytes of workspace for `max_partitions` partitions (per-partition max, sum and
 * normalised partial output, all fp32).  pa_decode with max_partitions == 1 needs no
 * workspace at all; pa_decode_partials / pa_merge always do.
 */
int64_t pa_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t head_dim,
                           int64_t max_partitions);

/*
 * Paged decode attention: one query token per sequence against its paged context.
 * Replaces: PagedAttention._decode_attention / _sdpa_decode_fallback
 *           (src/inference/attention.py:263-279, 317-382) when max_partitions == 1, and
 *           PartitionedPagedAttention._partitioned_decode_fallback with
 *           _compute_partition_attention + _merge_partitions
 *           (src/inference/attention.py:434-626) when max_partitions > 1.
 *
 * out[b, h, :] = softmax_j(scale * q[b,h,:] . K[b,j,h/G,:]) @ V[b,:,h/G,:] over the
 * first context_lens[b] tokens found through block_tables[b].  fp8 caches are
 * dequantised as fp8 / scale[slot].  Accumulation is fp32.
 *
 * max_partitions == 1: single pass, result written straight to `out`.
 * max_partitions  > 1: partition p of sequence b covers tokens
 *   [p*partition_size, min((p+1)*partition_size, context_len)); the last partition
 *   (p == max_partitions-1) absorbs whatever lies beyond it, so a context longer than
 *   max_partitions*partition_size is still computed exactly.  Per partition the
 *   kernel stores max (natural-log units), sum of exp and the locally normalised
 *   output into `workspace`; the merge reduction then writes `out`.
 *
 *   q, out               [batch, num_q_heads, head_dim], token stride in elements
 *   q_dtype              PA_DTYPE_F16 / BF16 / F32 (out has the same type)
 *   kv_dtype             PA_DTYPE_F16 / BF16 / FP8_E4M3
 *   k_scale, v_scale     required for fp8, ignored otherwise
 *   block_tables         rows bt_stride entries apart, table_width (<= bt_stride) of them valid
 *                        columns: a context that needs more columns than that re-reads the last
 *                        one instead of running off the row (pa_check_tables counts such rows)
 *   num_blocks           blocks in the pool (block ids are clamped to it)
 *   head_dim             64 or 128;  block_size a power of two >= 8
 *   num_q_heads          any multiple of num_kv_heads; all query heads of a KV head are served
 *                        by one workgroup (so its K/V rows leave HBM once) when the ratio is
 *                        1, 2, 4, 8 or 16, by ratio/4, ratio/2 or ratio workgroups otherwise
 *   partition_size       a multiple of 16 (ignored when max_partitions == 1)
 *   workspace            >= pa_workspace_bytes(...) bytes, 256-byte aligned
 *   waves_per_workgroup  0 = the launch's own choice, or 1, 2, 4, 8
 *   kv_heads_per_wave    0 = the launch's own choice (1 or 2), or 1, 2, 4, 8: adjacent KV heads
 *                        read by one wavefront, i.e. contiguous pieces of that many head rows per
 *                        token.  More than one needs num_q_heads / num_kv_heads <= 2 and a
 *                        num_kv_heads it divides; 4 and 8 also need a ratio of 2 and 4 or 8 waves
 *                        (PA_ERR_UNSUPPORTED otherwise).
 *   q_heads_per_wave     0 = the launch's own choice, or 1, 2, 4 (a divisor of the GQA ratio):
 *                        query heads of a KV head held in one wave's registers; the rest of the
 *                        ratio goes to groups of waves inside the workgroup (factors 2 and 4)
 *                        and, beyond that, to separate workgroups.  16 = the matrix kernel: up
 *                        to 16 query heads of a KV head (any ratio; wider groups in slices of 16)
 *                        as one MFMA operand, the launch's own choice from a ratio of 3 on; it
 *                        takes 2, 4 or 8 waves and kv_heads_per_wave 1, or 2 (of an even number
 *                        of KV heads, with 2 or 4 waves).
 *                        The result does not depend on any of the three.
 */
int pa_decode(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
              const void* v_cache, const float* k_scale, const float* v_scale, int kv_dtype,
              const int32_t* block_tables, int64_t bt_stride, int64_t table_width,
              const int32_t* context_lens, void* out, int64_t out_token_stride, int64_t batch,
              int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
              int64_t num_blocks, float scale, int64_t partition_size, int64_t max_partitions,
              void* workspace, int64_t workspace_bytes, int waves_per_workgroup,
              int kv_heads_per_wave, int q_heads_per_wave, void* stream);

/*
 * pa_decode for callers that cannot allocate device memory or hand over a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the partition
 * partials go to an array of PA_NOALLOC_SCRATCH_BYTES that is part of the library's device image,
 * one copy per GPU, held until the process ends.  Same arguments and same result, bit for bit,
 * as pa_decode without `workspace` / `workspace_bytes`; the call allocates and frees nothing.
 * A launch whose partials need more than the array holds (pa_workspace_bytes(batch, num_q_heads,
 * head_dim, max_partitions) > PA_NOALLOC_SCRATCH_BYTES) is refused with PA_ERR_WORKSPACE.
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two
 * streams, two threads) race on it and must be serialised by the caller; nothing an earlier
 * call left in it is ever read.
 * No counterpart in the reference (it allocates its partials as fresh tensors per call,
 * src/inference/attention.py:456-470).
 */
#define PA_NOALLOC_SCRATCH_BYTES (16 * 1024 * 1024)
int pa_decode_noalloc(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
                      const void* v_cache, const float* k_scale, const float* v_scale, int kv_dtype,
                      const int32_t* block_tables, int64_t bt_stride, int64_t table_width,
                      const int32_t* context_lens, void* out, int64_t out_token_stride,
                      int64_t batch, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                      int64_t block_size, int64_t num_blocks, float scale, int64_t partition_size,
                      int64_t max_partitions, int waves_per_workgroup, int kv_heads_per_wave,
                      int q_heads_per_wave, void* stream);

/*
 * First half of the partitioned decode only: fills `workspace` and does not merge.
 * Replaces: the loop over _compute_partition_attention
 *           (src/inference/attention.py:462-470, 519-589).
 * Workspace layout (fp32):  max [batch, num_q_heads, max_partitions]
 *                           sum [batch, num_q_heads, max_partitions]
 *                           out [batch, num_q_heads, max_partitions, head_dim]
 * Partition lse = max + log(sum).  Entries of partitions past the context are not written.
 */
int pa_decode_partials(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
                       const void* v_cache, const float* k_scale, const float* v_scale,
                       int kv_dtype, const int32_t* block_tables, int64_t bt_stride,
                       int64_t table_width, const int32_t* context_lens, int64_t batch,
                       int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                       int64_t block_size, int64_t num_blocks, float scale, int64_t partition_size,
                       int64_t max_partitions, void* workspace, int64_t workspace_bytes,
                       int waves_per_workgroup, int kv_heads_per_wave, int q_heads_per_wave,
                       void* stream);

/*
 * Partitioned decode for batches whose rows share prefixes as the same physical blocks (n samples
 * of one prompt, sequences forked from a cached prefix): partitions that lie wholly inside a
 * group's shared prefix are computed once for all the group's rows - their K and V leave HBM and
 * the L2 once per group instead of once per row - and every row's remaining partitions as usual;
 * the merge is pa_merge's.  Same result as pa_decode with the same partition_size.
 * Replaces: the same reference code as pa_decode (src/inference/attention.py:434-626); the
 * reference reads a shared block once per sequence that maps it (blocks carry a ref_count for
 * prefix sharing, src/inference/kv_cache.py:42-62, 190-210).
 * Arguments as pa_decode (partition_size > 0; the matrix kernel, one KV head per wave), plus:
 *   group_desc            device int32 [num_groups][4]: first, number of rows, shared partitions,
 *                         unused.  The first shared_partitions x partition_size tokens of every row
 *                         of a group must map to the same physical blocks as the group's first row,
 *                         and every row's context must hold them.  A group of 0 shared partitions
 *                         is empty (padding: a recorded HIP graph keeps num_groups fixed).
 *   group_rows            NULL: a group's rows are the consecutive batch rows first .. first + rows - 1.
 *                         Else device int32 [num_group_rows]: the group's rows are
 *                         group_rows[first .. first + rows - 1], any batch rows in any order.
 *   max_group_rows        most rows of any group; rows x (num_q_heads / num_kv_heads) <= 16
 *   max_shared_partitions most shared partitions of any group
 *   row_skip              device int32 [batch]: the row's group's shared partitions, 0 for rows of
 *                         no group
 *   max_own_partitions    most partitions any row computes itself:
 *                         >= ceil(context_len / partition_size) - row_skip[row] for every row
 * The launch trusts what the descriptors say is shared (pa_check_shared_prefix counts what is wrong
 * with them); indices read from them are clamped, so that a corrupt descriptor cannot fault.
 */
int pa_decode_shared_prefix(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
                            const void* v_cache, const float* k_scale, const float* v_scale,
                            int kv_dtype, const int32_t* block_tables, int64_t bt_stride,
                            int64_t table_width, const int32_t* context_lens, void* out,
                            int64_t out_token_stride, int64_t batch, int64_t num_q_heads,
                            int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                            int64_t num_blocks, float scale, int64_t partition_size,
                            int64_t max_partitions, void* workspace, int64_t workspace_bytes,
                            int waves_per_workgroup, const int32_t* group_desc, int64_t num_groups,
                            const int32_t* group_rows, int64_t num_group_rows,
                            int64_t max_group_rows, int64_t max_shared_partitions,
                            const int32_t* row_skip, int64_t max_own_partitions, void* stream);

/*
 * Debug aid for pa_decode_shared_prefix: counts, on the device, what is wrong with its descriptors.
 *   counts[0] += table entries inside a group's shared partitions that differ between a row and
 *                the group's first row (or lie beyond table_width)
 *   counts[1] += rows whose context is shorter than their group's shared tokens or whose row_skip
 *                is not their group's shared partitions; groups that reach outside the batch
 *   counts[2] += rows of no group with a non-zero row_skip, rows claimed by two groups
 * counts is a device int32[3] that the caller clears beforehand and reads afterwards.
 * No counterpart in the reference.
 */
int pa_check_shared_prefix(const int32_t* block_tables, int64_t bt_stride, int64_t table_width,
                           const int32_t* context_lens, int64_t batch, int64_t block_size,
                           int64_t partition_size, const int32_t* group_desc, int64_t num_groups,
                           const int32_t* group_rows, int64_t num_group_rows,
                           const int32_t* row_skip, int32_t* counts, void* stream);

/*
 * Merge reduction over partitions.
 * Replaces: PartitionedPagedAttention._merge_partitions (src/inference/attention.py:591-626).
 * out = sum_p w_p * out_p / sum_p w_p with w_p = sum_p * exp(max_p - max_all), over the
 * min(ceil(context_len/partition_size), max_partitions) partitions of each sequence.
 */
int pa_merge(const void* workspace, int64_t workspace_bytes, const int32_t* context_lens,
             void* out, int out_dtype, int64_t out_token_stride, int64_t batch,
             int64_t num_q_heads, int64_t head_dim, int64_t partition_size,
             int64_t max_partitions, void* stream);

/*
 * Chunked-prefill paged attention (MFMA): every new token of a sequence attends to the
 * cached prefix plus the new tokens up to itself, all read from the paged cache.
 * Replaces: PagedAttention._prefill_attention with block_tables set, i.e.
 *           flash_attn_varlen_func(..., causal=True, block_table=...)
 *           (src/inference/attention.py:240-261); with no prefix it equals
 *           _sdpa_prefill_fallback (src/inference/attention.py:281-315).
 * Row i of sequence s (i in [0, Lq_s)) sees keys [0, Lk_s - Lq_s + i] (bottom-right
 * aligned causal mask), Lq_s = cu_seqlens_q[s+1]-cu_seqlens_q[s],
 * Lk_s = cu_seqlens_k[s+1]-cu_seqlens_k[s] (cached + new tokens).
 *   q, out               [total_q_tokens, num_q_heads, head_dim]
 *   cu_seqlens_q/k       [num_seqs + 1] int32 (InferenceContext.cu_seqlens_q / cu_seqlens_k)
 *   block_tables         [num_seqs, bt_stride]; NULL = K/V are dense [total_k_tokens,
 *                        num_kv_heads, head_dim] tensors indexed by cu_seqlens_k (no prefix
 *                        hit: the reference then passes the new k, v themselves) and bt_stride
 *                        is their token stride in elements (0 = contiguous)
 *   kv_dtype             PA_DTYPE_F16 / BF16 / F32 / FP8_E4M3 (fp8 only with block_tables);
 *                        K/V and Q are multiplied as fp16 with fp32 accumulation
 *   head_dim             64 or 128;  block_size a power of two
 *   max_seqlen_q         upper bound of Lq_s (sizes the launch grid)
 *   scale                positive and finite
 *   waves_per_workgroup  0 = chosen per launch from the grid size, 4 (64 query tokens x 2 heads
 *                        per K/V tile) or 8 (128 x 2); the result does not depend on it
 */
int pa_prefill(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
               const void* v_cache, const float* k_scale, const float* v_scale, int kv_dtype,
               const int32_t* block_tables, int64_t bt_stride, const int32_t* cu_seqlens_q,
               const int32_t* cu_seqlens_k, void* out, int64_t out_token_stride,
               int64_t num_seqs, int64_t max_seqlen_q, int64_t num_q_heads,
               int64_t num_kv_heads, int64_t head_dim, int64_t block_size, int64_t num_blocks,
               float scale, int waves_per_workgroup, void* stream);

/*
 * fp8-e4m3fn -> fp32 conversion of n bytes (the in-register dequant step of the
 * attention kernels, exposed for checking the cache contents).
 * Replaces: `ki.to(torch.float16)` before the divide (src/inference/attention.py:361-362).
 */
int pa_fp8_e4m3_to_f32(const void* src, float* dst, int64_t n, void* stream);

/*
 * fp32 -> fp8-e4m3fn conversion of n values with the cache writer's rounding
 * (round-to-nearest-even, no saturation, NaN = 0x7F).
 * Replaces: `.to(torch.float8_e4m3fn)` (src/inference/attention.py:109-110).
 */
int pa_f32_to_fp8_e4m3(const float* src, void* dst, int64_t n, void* stream);

/*
 * Per-head RMSNorm of q and k, rotary embedding of both, and the paged cache write of k and v,
 * for num_tokens tokens in one launch.
 *   q [T, Hq, D], k, v [T, Hkv, D] in `dtype` (f16 / bf16 / f32), token strides in elements
 *   y = w * (x * rsqrt(mean(x^2) + eps)) per head row in fp32, rounded to `dtype`;
 *   then [y1, y2] -> [y1 cos - y2 sin, y2 cos + y1 sin] on the two halves of the row, with
 *   angle = float(positions[t]) * inv_freq[i], in fp32, rounded to `dtype`
 *   q_out [T, Hq, D] receives q; k_out (optional, may be NULL) a dense copy of k
 *   k_cache / v_cache [total_slots, Hkv, D]: slot_mapping[t] receives rotated k and raw v, as
 *   pa_kv_store (kv_dtype == dtype) or pa_kv_store_fp8 (kv_dtype == PA_DTYPE_FP8_E4M3, per-token
 *   scales to k_scale / v_scale) would write them; slot < 0 or >= total_slots: no cache write.
 *   k_cache == NULL: no cache write at all (v, v_cache, scales, slot_mapping unused).
 * head_dim 64 or 128; Hkv * D <= 2048; q, k, v, q_out, k_out rows, the weights and inv_freq 16-byte aligned.
 * Replaces: RMSNorm.forward on q and k (src/distributed/tensor_parallel.py:78-84, used at
 * :453-454), _apply_rotary_emb (:394-419, used at :457-464) and store_kv_cache
 * (src/inference/attention.py:44-183) of one attention layer.
 */
int pa_qk_norm_rope_store(const void* q, const void* k, const void* v, int dtype, int64_t q_token_stride,
                          int64_t k_token_stride, int64_t v_token_stride, const void* q_norm_weight,
                          const void* k_norm_weight, int weight_dtype, float eps, const float* inv_freq,
                          const int64_t* positions, void* q_out, int64_t q_out_token_stride, void* k_out,
                          int64_t k_out_token_stride, void* k_cache, void* v_cache, float* k_scale,
                          float* v_scale, int kv_dtype, const int32_t* slot_mapping, int64_t num_tokens,
                          int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t total_slots,
                          void* stream);

/*
 * One token per row of logits [batch, vocab] (f16 / bf16 / f32, rows row_stride elements apart),
 * written to out [batch] (int64).
 *   temperature <= 0: the index of the first maximum.
 *   otherwise: p_i = softmax(logits / temperature); with top_p < 1 a token stays iff the mass of
 *   the tokens with a strictly larger logit is <= top_p; the result is the first index j, in index
 *   order over the kept tokens, whose running sum of p exceeds uniforms[row] * (kept mass).
 *   uniforms: device fp32 [batch] in [0, 1), drawn by the caller (NULL allowed for greedy).
 * No sort, no host synchronisation; the call can be captured in a graph.
 * Replaces: ModelRunner.sample (src/inference/model_runner.py:590-634), whose multinomial draw is
 * replaced by the inverse-CDF lookup with caller-supplied uniform numbers.
 */
int pa_sample(const void* logits, int dtype, int64_t row_stride, int64_t batch, int64_t vocab,
              float temperature, float top_p, const float* uniforms, int64_t* out, void* stream);

/*
 * Gather the paged K and V of a batch into dense head-major tensors
 *     k_out, v_out  [batch, num_kv_heads, out_len, head_dim]   (same element type as the cache)
 * out[b, h, pos] = cache[slot(b, pos), h] for pos < context_lens[b] - len_offset, zeros after
 * that (and for positions whose table entry lies outside the table or the pool); slot(b, pos) =
 * block_tables[b][pos / block_size] * block_size + pos % block_size.  Bytes are moved as they are
 * (elem_bytes 1, 2 or 4; head_dim * elem_bytes a multiple of 16; 16-byte aligned bases).
 * Replaces: ModelRunner._load_kv_from_paged_cache (src/inference/model_runner.py:340-420), one
 * layer of it: the per-entry Python slot loop, the index gather, the zeroing of the padding and
 * the transposing copy.  len_offset = 1 there (the token being decoded is not part of the past).
 */
int pa_gather_kv(const void* k_cache, const void* v_cache, const int32_t* block_tables, int64_t bt_stride,
                 int64_t table_width, const int32_t* context_lens, int64_t len_offset, void* k_out, void* v_out,
                 int64_t batch, int64_t num_kv_heads, int64_t head_dim, int64_t elem_bytes, int64_t block_size,
                 int64_t num_blocks, int64_t out_len, void* stream);

/*
 * One decode step of a batch whose metadata stays on the device.  For every row r with
 * context_lens[r] > 0: if new_blocks (optional, int32 [batch], -1 = none) holds a block id for the
 * row it is stored at block_tables[r][context_lens[r] / block_size] (the block the new token
 * opens); then positions[r] = context_lens[r] (int64, the new token's index), slots[r] = its
 * cache slot from the row's table (-1 when outside the table or the pool), and context_lens[r]
 * grows by one, so that it counts the token being written as the attention kernels expect.
 * With next_tokens (optional, int64 [batch], e.g. the sampler's output of the step before) the
 * row's input_ids[r] becomes next_tokens[r] - unless fresh[r] (optional, int32 [batch]) is set:
 * a row admitted since the last step keeps the token its prefill produced, and the flag is cleared.
 * Rows with context_lens[r] <= 0 are inactive: slots[r] = -1, positions[r] = 0, nothing else changes.
 * Replaces: the per-step host loops and uploads of ModelRunner.prepare_decode and
 * _prepare_block_tables (src/inference/model_runner.py:542-588, 814-828: one Python assignment
 * per table entry and five fresh device tensors per step).
 */
int pa_decode_advance(int32_t* block_tables, int64_t bt_stride, int32_t* context_lens, int64_t* positions,
                      int32_t* slots, const int32_t* new_blocks, int64_t* input_ids, const int64_t* next_tokens,
                      int32_t* fresh, int64_t batch, int64_t table_width, int64_t block_size,
                      int64_t num_blocks, void* stream);

/*
 * One decoder block's residual add fused with the RMSNorm that follows it, one row per token:
 *     s = x + delta            rounded to `dtype` (skipped when delta == NULL: s = x)
 *     normed = weight * (s * rsqrt(mean(s^2) + eps))      fp32, rounded once to `dtype`
 * sum_out (optional, needs delta; may alias x or delta) receives s, the residual stream the next
 * block adds to.  Strides are row strides in elements; rows, weight and bases 16-byte aligned;
 * hidden a multiple of 8, at most 8192; weight may be f16, bf16 or f32.
 * Replaces: RMSNorm.forward (src/distributed/tensor_parallel.py:78-84) and the residual adds of
 * the block (tensor_parallel.py:640-651), seven plus one torch launches.
 */
int pa_add_rms_norm(const void* x, int64_t x_stride, const void* delta, int64_t delta_stride,
                    const void* weight, int weight_dtype, float eps, void* sum_out, int64_t sum_stride,
                    void* normed_out, int64_t normed_stride, int dtype, int64_t rows, int64_t hidden,
                    void* stream);

/*
 * out = silu(gate) * up, element-wise over [rows, width]; silu is rounded to `dtype` before the
 * product, as F.silu(gate) * up does.  gate and up may be the two halves of one packed
 * projection output (pass the same row stride).  width a multiple of 8, rows 16-byte aligned.
 * Replaces: the activation of the SwiGLU MLP (src/distributed/tensor_parallel.py:295-299).
 */
int pa_silu_mul(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride, void* out,
                int64_t out_stride, int dtype, int64_t rows, int64_t width, void* stream);

/*
 * Positions and cache slots of the tokens of one prefill step, on the device, from the step's two
 * cumulative length arrays (int32 [num_seqs + 1]: new tokens, and cached + new tokens, per sequence):
 * token t of chunk r gets positions[t] = cached_r + (t - cu_seqlens_q[r]) (int64) and
 * slots[t] = block_tables[row][positions[t] / block_size] * block_size + positions[t] % block_size
 * with row = row_index[r] (optional int32 [num_seqs]: the sequences' rows in a larger, device-resident
 * table of table_rows rows) or r.  slots may be NULL (no cache bound).  Tokens at or past
 * cu_seqlens_q[num_seqs] get position 0 and slot -1; a position past the table, a row outside it or
 * a block id outside [0, num_blocks) gives slot -1, which the KV writers skip.
 * Replaces: the position and slot loops of ModelRunner.prepare_prefill
 * (src/inference/model_runner.py:479-511) and the two uploads they end in.
 */
int pa_prefill_metadata(const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* block_tables,
                        int64_t bt_stride, const int32_t* row_index, int64_t* positions, int32_t* slots,
                        int64_t num_tokens, int64_t num_seqs, int64_t table_rows, int64_t table_width,
                        int64_t block_size, int64_t num_blocks, void* stream);

/*
 * slots[t] = block_tables[row(t)][positions[t] / block_size] * block_size + positions[t] % block_size
 * for num_tokens tokens, all on the device.  cu_seqlens_q == NULL: token t belongs to table row t
 * (one new token per sequence, num_tokens == num_rows).  Otherwise cu_seqlens_q is int32
 * [num_rows + 1] and row(t) is the sequence whose chunk [cu[r], cu[r+1]) holds t; tokens at or
 * past cu[num_rows] get -1.  positions is int64 (the reference's `positions` tensors are
 * torch.long).  A negative position, a position past table_width blocks, or a block id outside
 * [0, num_blocks) gives -1, which pa_kv_store / pa_kv_store_fp8 / pa_qk_norm_rope_store skip.
 * Replaces: the per-sequence host loop of ModelRunner.run_batch_decode
 * (src/inference/model_runner.py:670-682, two .item() reads per sequence) and the slot loops of
 * prepare_prefill (model_runner.py:493-511).
 */
int pa_slot_mapping(const int64_t* positions, const int32_t* cu_seqlens_q, const int32_t* block_tables,
                    int64_t bt_stride, int32_t* slots, int64_t num_tokens, int64_t num_rows,
                    int64_t table_width, int64_t block_size, int64_t num_blocks, void* stream);

/*
 * Copy whole cache blocks inside one pool tensor laid out [num_planes][num_blocks][block_bytes]
 * (planes plane_stride_bytes apart): for every plane and every pair i, block pairs[2i+1] := block
 * pairs[2i].  The K/V tensor of a BlockPool is one such tensor with 2 x layers planes, each fp8
 * scale tensor one with `layers` planes.  pairs is a device int32 array; pairs with an id outside
 * [0, num_blocks) or src == dst are skipped; no destination may be another pair's source.
 * Replaces: nothing the reference ships.  Its blocks carry a ref_count for prefix sharing
 * (src/inference/kv_cache.py:42-62, 195-212) but are never shared, and its K-sample path notes
 * that skipping the shared prompt needs block sharing / copying first
 * (src/inference/engine.py:1108-1113); this is the copy half of copy-on-write.
 */
int pa_copy_blocks(void* pool, int64_t num_planes, int64_t plane_stride_bytes, int64_t block_bytes,
                   int64_t num_blocks, const int32_t* pairs, int64_t num_pairs, void* stream);

/*
 * Debug aid for the caller side of the decode path.  The attention kernels never fault on a bad
 * table: they clamp block ids to the pool and table columns to table_width, which turns a
 * corrupt table into wrong numbers instead of an error.  This call counts, on the device, what a
 * decode launch over the same arguments would clamp:
 *   counts[0] += table entries in the first ceil(context_len / block_size) columns of a row
 *                that lie outside [0, num_blocks)
 *   counts[1] += rows whose context needs more than table_width columns
 * counts is a device int32[2] that the caller clears beforehand and reads afterwards.
 * No counterpart in the reference, whose host-side indexing raises on such input
 * (src/inference/attention.py:340-352).
 */
int pa_check_tables(const int32_t* block_tables, int64_t bt_stride, int64_t table_width,
                    const int32_t* context_lens, int64_t batch, int64_t block_size,
                    int64_t num_blocks, int32_t* counts, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* PAGED_ATTN_H_ */
