/*
 * pa_probes.h - C ABI of libpa_probes.so, the measuring aids of the MI355X paged-attention build.
 *
 * A library of its own beside libpaged_attn.so: nothing here is part of the product's interface or
 * has a counterpart in the reference.  bench.py and tests/test_gpu_probes.py load it; the product
 * never does.  Conventions (raw device pointers, int64 sizes, a HIP stream handle, negative PA_ERR_*
 * codes with pa_probes_last_error() holding the text) are those of paged_attn.h.
 */
#ifndef PA_PROBES_H_
#define PA_PROBES_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Message for the last negative return value on this thread ("" if none). */
const char* pa_probes_last_error(void);

/*
 * The launch of pa_decode_partials with the attention arithmetic taken out: the decode kernel
 * itself, built with its loads-only template flag.  Every K, V, scale and table load of the real
 * launch is issued from the same lanes in the same order and every loaded word is consumed (a
 * checksum lands in `workspace`), but no dot product, exponential or accumulation is done.  Its
 * duration is what the memory system needs for this access pattern alone - the ceiling the decode
 * kernel is measured against besides the nominal HBM rate.  Arguments as pa_decode_partials (no
 * scale factor); the workspace contents are meaningless afterwards.  Built for the vector kernel at
 * head_dim 128, 4-wave workgroups, 1 or 2 query heads per KV head and 1 or 2 KV heads per wave
 * (the shapes the headline launches take); anything else returns PA_ERR_UNSUPPORTED.
 */
int pa_decode_load_probe(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
                         const void* v_cache, const float* k_scale, const float* v_scale,
                         int kv_dtype, const int32_t* block_tables, int64_t bt_stride,
                         int64_t table_width, const int32_t* context_lens, int64_t batch,
                         int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                         int64_t block_size, int64_t num_blocks, int64_t partition_size,
                         int64_t max_partitions, void* workspace, int64_t workspace_bytes,
                         int waves_per_workgroup, int kv_heads_per_wave, int q_heads_per_wave,
                         void* stream);

/*
 * The rate the matrix pipe sustains.  Runs nothing but independent v_mfma_f32_32x32x16_f16 on every
 * SIMD (one workgroup of 8 waves per compute unit, `steps` x 16 products per wave) on operands taken
 * from `operands_f16` (num_operands >= 65536 fp16 values: constants, or the kind of data the
 * attention kernels see - the clocks of the part depend on how the operands toggle).  `sink`
 * receives one float per compute unit (sink_floats >= the device's compute units).  Returns the
 * number of floating-point operations of the launch (time it with events on `stream`), or a
 * negative error code.
 */
int64_t pa_mfma_rate_probe(const void* operands_f16, int64_t num_operands, int64_t steps, float* sink,
                           int64_t sink_floats, void* stream);

/*
 * The plain read rate of the GPU.  `groups` workgroups of 256 threads each stream their own
 * contiguous share of `bytes` bytes at `src` once (16-byte loads, four per lane in flight;
 * streaming != 0: non-temporal loads, the way the decode kernels read private K and V) and leave the
 * XOR of their words, folded to 32 bits, in sink[group] (sink_words >= groups).  Returns the number
 * of bytes read (bytes rounded down to 16 x groups), or a negative error code.
 */
int64_t pa_hbm_read_probe(const void* src, int64_t bytes, int64_t groups, int streaming, uint32_t* sink,
                          int64_t sink_words, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* PA_PROBES_H_ */
