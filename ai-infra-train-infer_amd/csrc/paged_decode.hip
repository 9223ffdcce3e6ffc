// Paged decode attention for gfx950: launch shaping, the merge reduction and the C entry points.
// The attention kernel itself is in paged_decode_kernel.hpp (instantiated per cache element type
// in paged_decode_f16.hip / _bf16.hip / _fp8.hip).
//
// Reference semantics: src/inference/attention.py:317-382 (single pass), :434-476 (partitioned
// driver), :519-589 (one partition) and :591-626 (merge).
#include "paged_decode_launch.hpp"

#include <stdio.h>

#include <mutex>

namespace pa {

// out = sum_p w_p out_p / sum_p w_p, w_p = sum_p * exp(max_p - max), over the partitions of one
// (batch row, query head) per workgroup.  A partition's partial output (head_dim floats) is read
// by head_dim / 4 lanes as 16-byte pieces, so the 256 threads of the workgroup work on several
// partitions at once ("slots": 8 at head_dim 128), each slot taking every slots-th partition in
// one pass with a running maximum, four independent loads in flight per thread; the slots are
// then combined through LDS.  (Before: one thread per element walking all partitions twice, 8.9 us
// for 53 partitions of 4 x 16 rows.)
constexpr int kMergeThreads = 256;
constexpr int kMergeUnroll = 4;

__global__ __launch_bounds__(kMergeThreads) void merge_partitions_kernel(
    const float* __restrict__ ws_max, const float* __restrict__ ws_sum, const float* __restrict__ ws_out,
    const int32_t* __restrict__ context_lens, void* out, int out_dtype, int64_t out_stride, int num_q_heads,
    int head_dim, int partition_size, int max_partitions) {
  __shared__ float4 s_acc[kMergeThreads];
  __shared__ float s_m[kMergeThreads], s_den[kMergeThreads];
  const int h = blockIdx.x;
  const int b = blockIdx.y;
  const int tid = threadIdx.x;
  const int ctx = context_lens[b];
  const int64_t o = b * out_stride + (int64_t)h * head_dim;
  if (ctx <= 0) {
    for (int d = tid; d < head_dim; d += kMergeThreads) store_from_f32(out, o + d, out_dtype, 0.0f);
    return;
  }
  const int np = min((ctx + partition_size - 1) / partition_size, max_partitions);
  const int lpp = head_dim >> 2;                 // lanes per partition row
  const int slots = kMergeThreads / lpp;
  const int slot = tid / lpp;
  const int ld = tid - slot * lpp;               // which 16-byte piece of the row
  const int64_t row0 = ((int64_t)b * num_q_heads + h) * max_partitions;
  float m = -INFINITY, den = 0.0f;
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  if (slot < slots) {
    for (int q0 = slot; q0 < np; q0 += slots * kMergeUnroll) {
      float pm[kMergeUnroll], ps[kMergeUnroll];
      float4 po[kMergeUnroll];
#pragma unroll
      for (int u = 0; u < kMergeUnroll; ++u) {
        const int q = q0 + u * slots;
        const bool live = q < np;
        const int64_t r = row0 + (live ? q : q0);
        pm[u] = live ? ws_max[r] : -INFINITY;
        ps[u] = live ? ws_sum[r] : 0.0f;
        po[u] = *(const float4*)(ws_out + r * head_dim + 4 * ld);
      }
#pragma unroll
      for (int u = 0; u < kMergeUnroll; ++u) {
        const float m_new = fmaxf(m, pm[u]);     // finite: partition q0 of this pass is live
        const float a = __expf(m - m_new);
        const float w = ps[u] * __expf(pm[u] - m_new);
        den = fmaf(den, a, w);
        acc.x = fmaf(acc.x, a, w * po[u].x);
        acc.y = fmaf(acc.y, a, w * po[u].y);
        acc.z = fmaf(acc.z, a, w * po[u].z);
        acc.w = fmaf(acc.w, a, w * po[u].w);
        m = m_new;
      }
    }
  }
  s_m[tid] = m;
  s_den[tid] = den;
  s_acc[tid] = acc;
  __syncthreads();
  if (slot != 0) return;
  const int used = min(slots, np);               // slots that saw a partition
  float mx = m;
  for (int i = 1; i < used; ++i) mx = fmaxf(mx, s_m[i * lpp + ld]);
  float d_all = 0.0f;
  float4 n_all = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  for (int i = 0; i < used; ++i) {
    const int t = i * lpp + ld;
    const float w = __expf(s_m[t] - mx);
    const float4 a = s_acc[t];
    d_all = fmaf(s_den[t], w, d_all);
    n_all.x = fmaf(a.x, w, n_all.x);
    n_all.y = fmaf(a.y, w, n_all.y);
    n_all.z = fmaf(a.z, w, n_all.z);
    n_all.w = fmaf(a.w, w, n_all.w);
  }
  const float inv = 1.0f / d_all;
  store_from_f32(out, o + 4 * ld, out_dtype, n_all.x * inv);
  store_from_f32(out, o + 4 * ld + 1, out_dtype, n_all.y * inv);
  store_from_f32(out, o + 4 * ld + 2, out_dtype, n_all.z * inv);
  store_from_f32(out, o + 4 * ld + 3, out_dtype, n_all.w * inv);
}

static int launch_merge(const float* ws_max, const float* ws_sum, const float* ws_out, const int32_t* context_lens,
                        void* out, int out_dtype, int64_t out_stride, int64_t batch, int64_t num_q_heads,
                        int64_t head_dim, int64_t partition_size, int64_t max_partitions, hipStream_t st) {
  hipLaunchKernelGGL(merge_partitions_kernel, dim3((unsigned)num_q_heads, (unsigned)batch), dim3(kMergeThreads), 0,
                     st, ws_max, ws_sum, ws_out, context_lens, out, out_dtype, out_stride, (int)num_q_heads,
                     (int)head_dim, (int)partition_size, (int)max_partitions);
  return PA_OK;
}

// Debug aid: counts what the attention kernels would silently clamp.  counts[0] = block-table
// entries inside a sequence's context that lie outside [0, num_blocks); counts[1] = sequences
// whose context needs more table columns than the table has.  One thread per table entry.
__global__ void check_tables_kernel(const int32_t* __restrict__ block_tables, int64_t bt_stride,
                                    int table_width, const int32_t* __restrict__ context_lens,
                                    int bs_log2, int num_blocks, int32_t* counts) {
  const int b = blockIdx.y;
  const int col = blockIdx.x * blockDim.x + threadIdx.x;
  const int ctx = context_lens[b];
  if (ctx <= 0) return;
  const int need = (ctx + (1 << bs_log2) - 1) >> bs_log2;
  if (col == 0 && need > table_width) atomicAdd(&counts[1], 1);
  if (col >= need || col >= table_width) return;
  const int id = block_tables[b * bt_stride + col];
  if (id < 0 || id >= num_blocks) atomicAdd(&counts[0], 1);
}

// Debug aid for shared-prefix launches: counts[0] = table entries of a group's shared partitions
// that differ between a row and the group's first row; counts[1] = rows whose context is shorter
// than the tokens their group shares, or whose row_skip differs from their group's shared
// partitions, and groups that reach outside the batch or the row list; counts[2] = rows that belong
// to no group but have a non-zero row_skip, or to two groups.
// One workgroup per group, one thread per shared table entry (strided).
__global__ void check_shared_prefix_kernel(const int32_t* __restrict__ block_tables, int64_t bt_stride,
                                           int table_width, const int32_t* __restrict__ context_lens,
                                           int batch, int bs_log2, int partition_size,
                                           const int32_t* __restrict__ group_desc, int num_groups,
                                           const int32_t* __restrict__ group_rows, int group_rows_len,
                                           const int32_t* __restrict__ row_skip, int32_t* counts) {
  const int gi = blockIdx.x;
  auto row_of = [&](int k, int m) { return group_rows ? group_rows[group_desc[4 * k] + m] : group_desc[4 * k] + m; };
  auto well_formed = [&](int k) {
    const int first = group_desc[4 * k], rows = group_desc[4 * k + 1];
    if (rows < 1 || first < 0 || group_desc[4 * k + 2] < 0) return false;
    return group_rows ? first + rows <= group_rows_len : first + rows <= batch;
  };
  if (gi == num_groups) {
    // rows outside every group must skip nothing; rows inside exactly one
    for (int b = threadIdx.x; b < batch; b += blockDim.x) {
      int owners = 0;
      for (int k = 0; k < num_groups; ++k) {
        if (!well_formed(k) || group_desc[4 * k + 2] == 0) continue;      // empty groups claim nothing
        for (int m = 0; m < group_desc[4 * k + 1]; ++m) owners += row_of(k, m) == b ? 1 : 0;
      }
      if ((owners == 0 && row_skip[b] != 0) || owners > 1) atomicAdd(&counts[2], 1);
    }
    return;
  }
  const int rows = group_desc[4 * gi + 1], parts = group_desc[4 * gi + 2];
  if (parts == 0) return;                                                   // an empty (padding) group
  const int shared_tokens = parts * partition_size;
  const int shared_blocks = (shared_tokens + (1 << bs_log2) - 1) >> bs_log2;
  if (!well_formed(gi)) {
    if (threadIdx.x == 0) atomicAdd(&counts[1], 1);
    return;
  }
  for (int m = 0; m < rows; ++m) {
    const int r = row_of(gi, m);
    if (r < 0 || r >= batch) {
      if (threadIdx.x == 0) atomicAdd(&counts[1], 1);
      return;
    }
  }
  const int lead = row_of(gi, 0);
  for (int m = threadIdx.x; m < rows; m += blockDim.x) {
    const int r = row_of(gi, m);
    if (context_lens[r] < shared_tokens || row_skip[r] != parts) atomicAdd(&counts[1], 1);
  }
  for (int e = threadIdx.x; e < shared_blocks * (rows - 1); e += blockDim.x) {
    const int m = 1 + e / shared_blocks, c = e % shared_blocks;
    if (c >= table_width || block_tables[row_of(gi, m) * bt_stride + c] != block_tables[lead * bt_stride + c])
      atomicAdd(&counts[0], 1);
  }
}

// ---- scratch of the entry point that allocates nothing ------------------------------------------
// Partition partials of pa_decode_noalloc.  The array's name is only a host-side handle; the
// device address is asked once per device and kept.
constexpr int64_t kNoAllocScratchBytes = PA_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
static void* g_scratch_ptr[kMaxDevices] = {};
static std::mutex g_scratch_mutex;

static int scratch_for_current_device(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(PA_ERR_LAUNCH, "pa_decode_noalloc: cannot tell the current device");
  void* ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (!ptr) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    ptr = g_scratch_ptr[dev];
    if (!ptr) {
      const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
      if (e != hipSuccess || !ptr) {
        char msg[160];
        snprintf(msg, sizeof(msg), "pa_decode_noalloc: hipGetSymbolAddress failed: HIP error %d (%s)",
                 (int)e, hipGetErrorString(e));
        return fail(PA_ERR_LAUNCH, msg);
      }
      __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
    }
  }
  *out = ptr;
  return PA_OK;
}

enum { kDecodeFull = 0, kDecodePartials = 1 };

// Shared argument checking + launch of the attention pass; kDecodeFull adds the reduction.
static int decode_impl(const char* who, const void* q, int q_dtype, int64_t q_token_stride,
                       const void* k_cache, const void* v_cache, const float* k_scale,
                       const float* v_scale, int kv_dtype, const int32_t* block_tables,
                       int64_t bt_stride, int64_t table_width, const int32_t* context_lens, void* out,
                       int64_t out_token_stride, int64_t batch, int64_t num_q_heads,
                       int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                       int64_t num_blocks, float scale, int64_t partition_size,
                       int64_t max_partitions, void* workspace, int64_t workspace_bytes,
                       int waves, int kv_heads_per_wave, int q_heads_per_wave, int mode,
                       void* stream, const SharedPrefix* shared = nullptr) {
  const bool merge = mode == kDecodeFull;
  DecodePlan plan;
  int rc = plan_decode(who, q, q_dtype, q_token_stride, k_cache, v_cache, k_scale, v_scale, kv_dtype,
                       block_tables, bt_stride, table_width, context_lens, out, out_token_stride, batch,
                       num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, scale, partition_size,
                       max_partitions, workspace, workspace_bytes, waves, kv_heads_per_wave,
                       q_heads_per_wave, merge, false, shared, &plan);
  if (rc != PA_OK || plan.empty) return rc;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(plan.grid);
  switch (plan.kv) {
    case KV_F16: rc = launch_decode_f16(plan.p, grid, plan.s, st); break;
    case KV_BF16: rc = launch_decode_bf16(plan.p, grid, plan.s, st); break;
    default: rc = launch_decode_fp8(plan.p, grid, plan.s, st); break;
  }
  if (rc != PA_OK) return rc;
  rc = check_launch(who);
  if (rc != PA_OK || plan.direct || !merge) return rc;
  launch_merge(plan.p.ws_max, plan.p.ws_sum, plan.p.ws_out, context_lens, out, q_dtype, out_token_stride, batch,
               num_q_heads, head_dim, plan.p.partition_size, plan.p.max_partitions, st);
  return check_launch(who);
}

}  // namespace pa

using namespace pa;

extern "C" int64_t pa_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t head_dim,
                                      int64_t max_partitions) {
  if (batch < 0 || num_q_heads < 0 || head_dim < 0) return 0;
  return ws_bytes(batch, num_q_heads, head_dim, max_partitions);
}

extern "C" int pa_decode(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
                         const void* v_cache, const float* k_scale, const float* v_scale,
                         int kv_dtype, const int32_t* block_tables, int64_t bt_stride,
                         int64_t table_width, const int32_t* context_lens, void* out,
                         int64_t out_token_stride, int64_t batch, int64_t num_q_heads,
                         int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                         int64_t num_blocks, float scale, int64_t partition_size,
                         int64_t max_partitions, void* workspace, int64_t workspace_bytes,
                         int waves_per_workgroup, int kv_heads_per_wave, int q_heads_per_wave,
                         void* stream) {
  return decode_impl("pa_decode", q, q_dtype, q_token_stride, k_cache, v_cache, k_scale, v_scale,
                     kv_dtype, block_tables, bt_stride, table_width, context_lens, out,
                     out_token_stride, batch, num_q_heads, num_kv_heads, head_dim, block_size,
                     num_blocks, scale, partition_size, max_partitions, workspace, workspace_bytes,
                     waves_per_workgroup, kv_heads_per_wave, q_heads_per_wave, kDecodeFull, stream);
}

extern "C" int pa_decode_noalloc(const void* q, int q_dtype, int64_t q_token_stride,
                                 const void* k_cache, const void* v_cache, const float* k_scale,
                                 const float* v_scale, int kv_dtype, const int32_t* block_tables,
                                 int64_t bt_stride, int64_t table_width, const int32_t* context_lens,
                                 void* out, int64_t out_token_stride, int64_t batch,
                                 int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                 int64_t block_size, int64_t num_blocks, float scale,
                                 int64_t partition_size, int64_t max_partitions,
                                 int waves_per_workgroup, int kv_heads_per_wave, int q_heads_per_wave,
                         void* stream) {
  void* ws = nullptr;
  if (max_partitions > 1) {
    if (batch < 0 || num_q_heads <= 0 || head_dim <= 0)
      return fail(PA_ERR_BAD_ARG, "pa_decode_noalloc: negative or zero size");
    const int64_t need = ws_bytes(batch, num_q_heads, head_dim, max_partitions);
    if (need > kNoAllocScratchBytes) {
      char msg[200];
      snprintf(msg, sizeof(msg),
               "pa_decode_noalloc: partials of this launch need %lld bytes, the built-in scratch holds %lld "
               "(use pa_decode with a caller-owned workspace)",
               (long long)need, (long long)kNoAllocScratchBytes);
      return fail(PA_ERR_WORKSPACE, msg);
    }
    const int rc = scratch_for_current_device(&ws);
    if (rc != PA_OK) return rc;
  }
  // Every partial the merge reads is written by this launch's own attention pass, so nothing
  // left in the array by an earlier call needs clearing.
  return decode_impl("pa_decode_noalloc", q, q_dtype, q_token_stride, k_cache, v_cache, k_scale,
                     v_scale, kv_dtype, block_tables, bt_stride, table_width, context_lens, out,
                     out_token_stride, batch, num_q_heads, num_kv_heads, head_dim, block_size,
                     num_blocks, scale, partition_size, max_partitions, ws,
                     ws ? kNoAllocScratchBytes : 0, waves_per_workgroup, kv_heads_per_wave, q_heads_per_wave, kDecodeFull, stream);
}

extern "C" int pa_decode_partials(const void* q, int q_dtype, int64_t q_token_stride,
                                  const void* k_cache, const void* v_cache, const float* k_scale,
                                  const float* v_scale, int kv_dtype, const int32_t* block_tables,
                                  int64_t bt_stride, int64_t table_width, const int32_t* context_lens,
                                  int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                  int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                  float scale, int64_t partition_size, int64_t max_partitions,
                                  void* workspace, int64_t workspace_bytes, int waves_per_workgroup,
                                  int kv_heads_per_wave, int q_heads_per_wave, void* stream) {
  return decode_impl("pa_decode_partials", q, q_dtype, q_token_stride, k_cache, v_cache, k_scale,
                     v_scale, kv_dtype, block_tables, bt_stride, table_width, context_lens, nullptr,
                     0, batch, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, scale,
                     partition_size, max_partitions, workspace, workspace_bytes,
                     waves_per_workgroup, kv_heads_per_wave, q_heads_per_wave, kDecodePartials, stream);
}

extern "C" int pa_decode_shared_prefix(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
                                       const void* v_cache, const float* k_scale, const float* v_scale,
                                       int kv_dtype, const int32_t* block_tables, int64_t bt_stride,
                                       int64_t table_width, const int32_t* context_lens, void* out,
                                       int64_t out_token_stride, int64_t batch, int64_t num_q_heads,
                                       int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                                       int64_t num_blocks, float scale, int64_t partition_size,
                                       int64_t max_partitions, void* workspace, int64_t workspace_bytes,
                                       int waves_per_workgroup, const int32_t* group_desc,
                                       int64_t num_groups, const int32_t* group_rows,
                                       int64_t num_group_rows, int64_t max_group_rows,
                                       int64_t max_shared_partitions, const int32_t* row_skip,
                                       int64_t max_own_partitions, void* stream) {
  if (group_rows && (num_group_rows < 0 || num_group_rows > 0x7fffffff))
    return fail(PA_ERR_BAD_ARG, "pa_decode_shared_prefix: num_group_rows out of range");
  const SharedPrefix sp = {group_desc, group_rows, group_rows ? num_group_rows : 0, num_groups, max_group_rows,
                           max_shared_partitions, row_skip, max_own_partitions};
  return decode_impl("pa_decode_shared_prefix", q, q_dtype, q_token_stride, k_cache, v_cache, k_scale,
                     v_scale, kv_dtype, block_tables, bt_stride, table_width, context_lens, out,
                     out_token_stride, batch, num_q_heads, num_kv_heads, head_dim, block_size,
                     num_blocks, scale, partition_size, max_partitions, workspace, workspace_bytes,
                     waves_per_workgroup, 0, 0, kDecodeFull, stream, &sp);
}

extern "C" int pa_check_shared_prefix(const int32_t* block_tables, int64_t bt_stride, int64_t table_width,
                                      const int32_t* context_lens, int64_t batch, int64_t block_size,
                                      int64_t partition_size, const int32_t* group_desc,
                                      int64_t num_groups, const int32_t* group_rows,
                                      int64_t num_group_rows, const int32_t* row_skip, int32_t* counts,
                                      void* stream) {
  if (batch < 0 || bt_stride < 0 || table_width < 0 || num_groups < 0 || partition_size <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_check_shared_prefix: negative or zero size");
  if (!counts) return fail(PA_ERR_BAD_ARG, "pa_check_shared_prefix: null pointer");
  const int bs_log2 = ilog2_exact(block_size);
  if (bs_log2 < 0) return fail(PA_ERR_UNSUPPORTED, "pa_check_shared_prefix: block_size must be a power of two");
  if (batch == 0) return PA_OK;
  if (!block_tables || !context_lens || !row_skip || (num_groups > 0 && !group_desc))
    return fail(PA_ERR_BAD_ARG, "pa_check_shared_prefix: null pointer");
  if (batch > 0x7fffffff || table_width > 0x7fffffff || num_groups >= 0x7fffffff || partition_size > 0x7fffffff ||
      num_group_rows < 0 || num_group_rows > 0x7fffffff)
    return fail(PA_ERR_UNSUPPORTED, "pa_check_shared_prefix: batch, table or group count too large for one launch");
  hipLaunchKernelGGL(check_shared_prefix_kernel, dim3((unsigned)num_groups + 1), dim3(256), 0,
                     (hipStream_t)stream, block_tables, bt_stride, (int)table_width, context_lens,
                     (int)batch, bs_log2, (int)partition_size, group_desc, (int)num_groups, group_rows,
                     group_rows ? (int)num_group_rows : 0, row_skip, counts);
  return check_launch("pa_check_shared_prefix");
}

extern "C" int pa_merge(const void* workspace, int64_t workspace_bytes, const int32_t* context_lens,
                        void* out, int out_dtype, int64_t out_token_stride, int64_t batch,
                        int64_t num_q_heads, int64_t head_dim, int64_t partition_size,
                        int64_t max_partitions, void* stream) {
  if (batch < 0 || num_q_heads <= 0 || head_dim <= 0 || max_partitions < 1 || partition_size <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_merge: bad size");
  if (batch == 0) return PA_OK;
  if (!workspace || !context_lens || !out) return fail(PA_ERR_BAD_ARG, "pa_merge: null pointer");
  if (head_dim > 1024 || head_dim % 4 != 0) return fail(PA_ERR_UNSUPPORTED, "pa_merge: head_dim must be a multiple of 4, at most 1024");
  if (num_q_heads > 65535 || max_partitions > 0x7fffffff || partition_size > 0x7fffffff)
    return fail(PA_ERR_UNSUPPORTED, "pa_merge: head count, partition count or partition size too large");
  if (out_dtype != PA_DTYPE_F16 && out_dtype != PA_DTYPE_BF16 && out_dtype != PA_DTYPE_F32)
    return fail(PA_ERR_UNSUPPORTED, "pa_merge: out_dtype must be f16, bf16 or f32");
  if (workspace_bytes < ws_bytes(batch, num_q_heads, head_dim, max_partitions))
    return fail(PA_ERR_WORKSPACE, "pa_merge: workspace too small");
  if (!aligned16(workspace)) return fail(PA_ERR_BAD_ARG, "pa_merge: workspace must be 16-byte aligned");
  if (batch > 65535) return fail(PA_ERR_UNSUPPORTED, "pa_merge: batch too large");
  const Workspace w = ws_split(const_cast<void*>(workspace), batch, num_q_heads, max_partitions);
  launch_merge(w.mx, w.sum, w.out, context_lens, out, out_dtype, out_token_stride, batch, num_q_heads, head_dim,
               partition_size, max_partitions, (hipStream_t)stream);
  return check_launch("pa_merge");
}

extern "C" int pa_check_tables(const int32_t* block_tables, int64_t bt_stride, int64_t table_width,
                               const int32_t* context_lens, int64_t batch, int64_t block_size,
                               int64_t num_blocks, int32_t* counts, void* stream) {
  if (batch < 0 || bt_stride < 0 || table_width < 0 || num_blocks <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_check_tables: negative or zero size");
  if (!counts) return fail(PA_ERR_BAD_ARG, "pa_check_tables: null pointer");
  const int bs_log2 = ilog2_exact(block_size);
  if (bs_log2 < 0) return fail(PA_ERR_UNSUPPORTED, "pa_check_tables: block_size must be a power of two");
  if (batch == 0) return PA_OK;
  if (!block_tables || !context_lens) return fail(PA_ERR_BAD_ARG, "pa_check_tables: null pointer");
  if (batch > 65535 || table_width > 0x7fffffff || num_blocks > 0x7fffffff)
    return fail(PA_ERR_UNSUPPORTED, "pa_check_tables: batch, table or pool too large for one launch");
  const unsigned gx = (unsigned)((table_width + 255) / 256 > 0 ? (table_width + 255) / 256 : 1);
  hipLaunchKernelGGL(check_tables_kernel, dim3(gx, (unsigned)batch), dim3(256), 0, (hipStream_t)stream,
                     block_tables, bt_stride, (int)table_width, context_lens, bs_log2, (int)num_blocks,
                     counts);
  return check_launch("pa_check_tables");
}
