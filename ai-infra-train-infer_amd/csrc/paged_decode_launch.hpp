// Argument checking and launch shaping of a paged decode launch, shared by the entry points of the
// library (paged_decode.hip) and by the loads-only measuring build of the same kernel
// (probes/decode_load_probe.hip): both must cut a launch the same way.
//
// Reference semantics: src/inference/attention.py:317-382 (single pass), :434-476 (partitioned
// driver).
#pragma once

#include "paged_decode_kernel.hpp"

#include <stdio.h>

namespace pa {

// CUs of the current device (per device, asked once).
inline int compute_units() {
  static int cached[kMaxDevices] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
  }
  return n;
}

struct Workspace {
  float* mx;
  float* sum;
  float* out;
};

inline int64_t ws_bytes(int64_t batch, int64_t hq, int64_t d, int64_t maxp) {
  if (maxp < 1) maxp = 1;
  const int64_t rows = batch * hq * maxp;
  // max and sum are padded to a 256-byte boundary so the partial outputs stay 16-byte aligned
  const int64_t scalars = ((rows * 4 + 255) / 256) * 256;
  return 2 * scalars + rows * d * 4;
}

inline Workspace ws_split(void* ws, int64_t batch, int64_t hq, int64_t maxp) {
  const int64_t rows = batch * hq * maxp;
  const int64_t scalars = ((rows * 4 + 255) / 256) * 256;
  Workspace w;
  w.mx = (float*)ws;
  w.sum = (float*)((uint8_t*)ws + scalars);
  w.out = (float*)((uint8_t*)ws + 2 * scalars);
  return w;
}

inline int ilog2_exact(int64_t v) {
  if (v <= 0 || (v & (v - 1)) != 0) return -1;
  int l = 0;
  while ((int64_t(1) << l) < v) ++l;
  return l;
}

// What pa_decode_shared_prefix adds to a partitioned launch.
struct SharedPrefix {
  const int32_t* group_desc;
  const int32_t* group_rows;
  int64_t num_group_rows;
  int64_t num_groups;
  int64_t max_group_rows;
  int64_t max_shared_partitions;
  const int32_t* row_skip;
  int64_t max_own_partitions;
};

constexpr int kMatrixPath = 16;            // q_heads_per_wave value that names the MFMA kernel
constexpr int kMatrixPathFromRatio = 3;     // GQA ratio from which the automatic choice takes it

// A checked and shaped launch: kernel arguments, template selection and grid.
struct DecodePlan {
  DecodeParams p;
  DecodeShape s;
  unsigned grid;
  int kv;           // KV_F16 / KV_BF16 / KV_FP8
  bool direct;      // single pass straight into `out`: no partials, no merge
  bool empty;       // batch == 0: nothing to launch
};

// Checks the arguments of a decode launch and decides how it is cut.  `merge`: the launch is
// followed by the merge reduction (an output is required); `vector_only`: never the matrix path
// (the loads-only build follows the vector kernel).  Returns PA_OK or an error code with the
// thread's error text set.
inline int plan_decode(const char* who, const void* q, int q_dtype, int64_t q_token_stride,
                       const void* k_cache, const void* v_cache, const float* k_scale,
                       const float* v_scale, int kv_dtype, const int32_t* block_tables,
                       int64_t bt_stride, int64_t table_width, const int32_t* context_lens, void* out,
                       int64_t out_token_stride, int64_t batch, int64_t num_q_heads,
                       int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                       int64_t num_blocks, float scale, int64_t partition_size,
                       int64_t max_partitions, void* workspace, int64_t workspace_bytes,
                       int waves, int kv_heads_per_wave, int q_heads_per_wave, bool merge,
                       bool vector_only, const SharedPrefix* shared, DecodePlan* plan) {
  char msg[256];
#define PA_FAIL(code, text)                         \
  do {                                              \
    snprintf(msg, sizeof(msg), "%s: %s", who, text); \
    return fail(code, msg);                         \
  } while (0)
  plan->empty = false;
  if (batch < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 ||
      num_blocks <= 0 || bt_stride < 0 || table_width < 0)
    PA_FAIL(PA_ERR_BAD_ARG, "negative or zero size");
  if (batch == 0) {
    plan->empty = true;
    return PA_OK;
  }
  if (!q || !k_cache || !v_cache || !block_tables || !context_lens)
    PA_FAIL(PA_ERR_BAD_ARG, "null pointer");
  if (merge && !out) PA_FAIL(PA_ERR_BAD_ARG, "null output");
  if (table_width > bt_stride && batch > 1) PA_FAIL(PA_ERR_BAD_ARG, "table_width larger than the row stride");
  if (table_width > 0x7fffffff) PA_FAIL(PA_ERR_BAD_ARG, "table_width too large");
  if (q_dtype != PA_DTYPE_F16 && q_dtype != PA_DTYPE_BF16 && q_dtype != PA_DTYPE_F32)
    PA_FAIL(PA_ERR_UNSUPPORTED, "q_dtype must be f16, bf16 or f32");
  int kv;
  switch (kv_dtype) {
    case PA_DTYPE_F16: kv = KV_F16; break;
    case PA_DTYPE_BF16: kv = KV_BF16; break;
    case PA_DTYPE_FP8_E4M3: kv = KV_FP8; break;
    default: PA_FAIL(PA_ERR_UNSUPPORTED, "kv_dtype must be f16, bf16 or fp8-e4m3");
  }
  if (kv == KV_FP8 && (!k_scale || !v_scale))
    PA_FAIL(PA_ERR_BAD_ARG, "fp8 cache needs k_scale and v_scale");
  if (kv == KV_FP8 && (!aligned16(k_scale) || !aligned16(v_scale)))
    PA_FAIL(PA_ERR_BAD_ARG, "k_scale and v_scale must be 16-byte aligned");
  if (head_dim != 64 && head_dim != 128) PA_FAIL(PA_ERR_UNSUPPORTED, "head_dim must be 64 or 128");
  if (num_q_heads % num_kv_heads != 0)
    PA_FAIL(PA_ERR_BAD_ARG, "num_q_heads must be a multiple of num_kv_heads");
  const int bs_log2 = ilog2_exact(block_size);
  if (bs_log2 < 3) PA_FAIL(PA_ERR_UNSUPPORTED, "block_size must be a power of two >= 8");
  if (!aligned16(k_cache) || !aligned16(v_cache))
    PA_FAIL(PA_ERR_BAD_ARG, "caches must be 16-byte aligned");
  if (q_token_stride < num_q_heads * head_dim || (out && out_token_stride < num_q_heads * head_dim))
    PA_FAIL(PA_ERR_BAD_ARG, "token stride smaller than num_q_heads*head_dim");
  if (batch > 65535 || num_blocks > 0x7fffffff || num_q_heads > 65535)
    PA_FAIL(PA_ERR_UNSUPPORTED, "batch or head count too large for one launch");
  if (max_partitions < 1) max_partitions = 1;
  if (max_partitions > 65535) PA_FAIL(PA_ERR_UNSUPPORTED, "max_partitions > 65535");
  if (waves != 0 && waves != 1 && waves != 2 && waves != 4 && waves != 8)
    PA_FAIL(PA_ERR_BAD_ARG, "waves_per_workgroup must be 0 (automatic), 1, 2, 4 or 8");
  if (kv_heads_per_wave != 0 && kv_heads_per_wave != 1 && kv_heads_per_wave != 2 &&
      kv_heads_per_wave != 4 && kv_heads_per_wave != 8)
    PA_FAIL(PA_ERR_BAD_ARG, "kv_heads_per_wave must be 0 (automatic), 1, 2, 4 or 8");
  if (q_heads_per_wave != 0 && q_heads_per_wave != 1 && q_heads_per_wave != 2 && q_heads_per_wave != 4 &&
      q_heads_per_wave != kMatrixPath)
    PA_FAIL(PA_ERR_BAD_ARG, "q_heads_per_wave must be 0 (automatic), 1, 2, 4 or 16 (the matrix path)");
  const bool direct = merge && max_partitions == 1 && !shared;
  if (shared) {
    if (!shared->group_desc || !shared->row_skip) PA_FAIL(PA_ERR_BAD_ARG, "null group descriptors");
    if (shared->num_groups < 0 || shared->num_groups > 0x7fffffff || shared->max_group_rows < 1 ||
        shared->max_shared_partitions < 0 || shared->max_shared_partitions > max_partitions ||
        shared->max_own_partitions < 1 || shared->max_own_partitions > max_partitions)
      PA_FAIL(PA_ERR_BAD_ARG, "group counts out of range");
    if (partition_size <= 0) PA_FAIL(PA_ERR_BAD_ARG, "a shared-prefix launch is a partitioned launch: partition_size > 0");
    if ((num_q_heads / num_kv_heads) * shared->max_group_rows > kMatrixPath)
      PA_FAIL(PA_ERR_UNSUPPORTED, "rows per group x query heads per KV head must not exceed 16");
    if (kv_heads_per_wave > 1 || (q_heads_per_wave != 0 && q_heads_per_wave != kMatrixPath) || waves == 1)
      PA_FAIL(PA_ERR_UNSUPPORTED, "a shared-prefix launch runs on the matrix path with one KV head per wave");
  }
  if (!direct) {
    if ((max_partitions > 1 || shared) && (partition_size <= 0 || partition_size % 16 != 0))
      PA_FAIL(PA_ERR_UNSUPPORTED, "partition_size must be a positive multiple of 16");
    const int64_t need = ws_bytes(batch, num_q_heads, head_dim, max_partitions);
    if (!workspace || workspace_bytes < need) PA_FAIL(PA_ERR_WORKSPACE, "workspace missing or too small");
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
      PA_FAIL(PA_ERR_BAD_ARG, "workspace must be 256-byte aligned");
    if (partition_size > 0x7fffffff) PA_FAIL(PA_ERR_BAD_ARG, "partition_size too large");
  }

  // ---- how the query group of a KV head is spread over registers, waves and workgroups ----------
  // gc query heads in a wave's registers; qs groups of waves over the same tokens when the group
  // is wider than that; whatever is left over (ratios with a factor other than 2) goes to
  // separate workgroups, which then read the KV head once each.
  const int g = (int)(num_q_heads / num_kv_heads);
  DecodeShape& s = plan->s;
  s.head_dim = (int)head_dim;
  int slices;                                 // workgroups per KV head
  // The matrix path (paged_decode_mfma_kernel.hpp) takes up to 16 query heads of a KV head as one
  // MFMA operand: the choice from a GQA ratio of 3 on, where the vector kernel's arithmetic per
  // loaded byte starts to cost more than the loads (batch 64 x 4096 tokens, fp16 / fp8 cache: ratio 4
  // 187 / 103 us against 195 / 142 us, ratio 8 187 / 103 against 239 / 257, ratio 2 182 / 100.5 against 179 / 100).
  bool matrix = q_heads_per_wave == kMatrixPath || shared != nullptr;
  if (q_heads_per_wave == 0 && g >= kMatrixPathFromRatio && !vector_only && kv_heads_per_wave <= 2 &&
      (waves == 0 || waves >= 2) && !(kv_heads_per_wave == 2 && (waves == 8 || num_kv_heads % 2 != 0)))
    matrix = true;
  if (matrix) {
    if (vector_only) PA_FAIL(PA_ERR_UNSUPPORTED, "the loads-only build follows the vector kernel: q_heads_per_wave 1, 2 or 4");
    if (kv_heads_per_wave > 2 || (kv_heads_per_wave == 2 && num_kv_heads % 2 != 0))
      PA_FAIL(PA_ERR_UNSUPPORTED, "the matrix path takes one KV head per wave, or two of an even number");
    if (waves == 1 || (kv_heads_per_wave == 2 && waves == 8))
      PA_FAIL(PA_ERR_UNSUPPORTED, "the matrix path takes 2, 4 or 8 waves per workgroup with one KV head per wave, 2 or 4 with two");
    s.gc = kMatrixPath;
    s.qs = 1;
    slices = (g + kMatrixPath - 1) / kMatrixPath;
    // One KV head per wave.  4-wave workgroups (two share a CU) are the best or within 3 % of the best
    // shape from batch 8 x 320 to batch 256 x 1k tokens; launches with fewer workgroups than CUs put
    // 8 waves on the CUs they do reach.  Two heads per wave (256-byte pieces of an fp8 row, 32 KiB of
    // LDS per wave, so one 4-wave workgroup per CU) pay in one case only: an fp8 cache and a halved
    // grid that is just one workgroup per CU (batch 64 x 8 KV heads: 103-105 against 112-115 us);
    // with fewer workgroups they idle CUs, with more the second round costs what the pieces save.
    s.hpw = kv_heads_per_wave == 2 ? 2 : 1;
    const int64_t cus = compute_units();
    const int64_t unpaired = num_kv_heads * slices * max_partitions * batch;
    if (kv_heads_per_wave == 0 && kv == KV_FP8 && num_kv_heads % 2 == 0 && !shared && (waves == 0 || waves == 4) &&
        unpaired / 2 <= cus && unpaired / 2 * 10 >= cus * 9)
      s.hpw = 2;
    if (waves != 0) {
      s.waves = waves;
    } else {
      s.waves = (s.hpw == 1 && unpaired < cus && !shared) ? 8 : 4;
    }
  } else {
    if (q_heads_per_wave != 0) {
      if (g % q_heads_per_wave != 0) PA_FAIL(PA_ERR_UNSUPPORTED, "q_heads_per_wave must divide num_q_heads / num_kv_heads");
      s.gc = q_heads_per_wave;
    } else {
      s.gc = (g % 4 == 0) ? 4 : (g % 2 == 0) ? 2 : 1;
    }
    const int rest = g / s.gc;
    const int split_waves = s.gc == 4 ? 4 : 8;
    s.qs = 1;
    if (s.gc >= 2 && rest % 2 == 0 && (waves == 0 || waves == split_waves)) s.qs = (rest % 4 == 0) ? 4 : 2;
    slices = rest / s.qs;
    s.waves = s.qs > 1 ? split_waves : (waves == 0 ? 4 : waves);
    // Several adjacent KV heads per wave need each KV head's query group whole in the wave.
    const bool can_share = g == s.gc && s.gc <= 2;
    s.hpw = 1;
    if (kv_heads_per_wave > 1) {
      if (!can_share || num_kv_heads % kv_heads_per_wave != 0 ||
          (kv_heads_per_wave > 2 && (s.gc != 2 || (s.waves != 4 && s.waves != 8))))
        PA_FAIL(PA_ERR_UNSUPPORTED, "kv_heads_per_wave does not fit this head layout");
      s.hpw = kv_heads_per_wave;
    } else if (kv_heads_per_wave == 0 && can_share && num_kv_heads % 2 == 0) {
      // Two heads per wave when halving the workgroups does not add a round of them over the CUs: a
      // CU streams at a fixed rate however many workgroups it hosts, the launch takes as long as
      // its busiest CU, and fewer, longer-lived workgroups stream better (185 -> 178 us at batch 64 /
      // ctx 4096, fp16; rows of 128 bytes or less gain another 10% from being read as 256-byte
      // pieces).  With a workgroup or less per CU pairing would only idle CUs.
      const int64_t cus = compute_units();
      const int64_t wgs = num_kv_heads * max_partitions * batch;      // unpaired
      const int64_t rounds = (wgs + cus - 1) / cus, paired_rounds = (wgs + 2 * cus - 1) / (2 * cus);
      if (wgs >= 8 * cus || 2 * paired_rounds <= rounds) s.hpw = 2;
    }
  }

  DecodeParams& p = plan->p;
  p.q = q;
  p.q_stride = q_token_stride;
  p.k_cache = (const uint8_t*)k_cache;
  p.v_cache = (const uint8_t*)v_cache;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.block_tables = block_tables;
  p.bt_stride = bt_stride;
  p.table_width = (int)table_width;
  p.context_lens = context_lens;
  p.out = out;
  p.out_stride = out_token_stride;
  p.q_dtype = q_dtype;
  p.num_q_heads = (int)num_q_heads;
  p.num_kv_heads = (int)num_kv_heads;
  p.bs_log2 = bs_log2;
  p.num_blocks = (int)num_blocks;
  p.partition_size = (int)partition_size;
  p.max_partitions = (int)max_partitions;
  p.direct_out = direct ? 1 : 0;
  p.scale_log2e = scale * 1.4426950408889634f;
  p.ws_max = p.ws_sum = p.ws_out = nullptr;
  if (!direct) {
    const Workspace w = ws_split(workspace, batch, num_q_heads, max_partitions);
    p.ws_max = w.mx;
    p.ws_sum = w.sum;
    p.ws_out = w.out;
  }
  p.inner = (int)(num_kv_heads / s.hpw) * slices;
  p.xcd_rows = (kv == KV_FP8 && !shared && p.inner > 1 && (batch * max_partitions) % 8 == 0) ? 1 : 0;
  p.batch = (int)batch;
  p.group_desc = nullptr;
  p.group_rows = nullptr;
  p.group_rows_len = 0;
  p.row_skip = nullptr;
  p.num_groups = p.num_prefix_wgs = p.prefix_parts = p.suffix_parts = 0;
  int64_t wgs = batch * max_partitions * p.inner;
  if (shared) {
    const int64_t prefix_wgs = shared->num_groups * shared->max_shared_partitions * p.inner;
    wgs = prefix_wgs + batch * shared->max_own_partitions * p.inner;
    if (prefix_wgs > 0x7fffffff) PA_FAIL(PA_ERR_UNSUPPORTED, "too many workgroups for one launch");
    p.group_desc = shared->group_desc;
    p.group_rows = shared->group_rows;
    p.group_rows_len = (int)shared->num_group_rows;
    p.row_skip = shared->row_skip;
    p.num_groups = (int)shared->num_groups;
    p.num_prefix_wgs = (int)prefix_wgs;
    p.prefix_parts = (int)shared->max_shared_partitions;
    p.suffix_parts = (int)shared->max_own_partitions;
  }
  if (wgs > 0x7fffffff) PA_FAIL(PA_ERR_UNSUPPORTED, "too many workgroups for one launch");
#undef PA_FAIL
  plan->grid = (unsigned)wgs;
  plan->kv = kv;
  plan->direct = direct;
  return PA_OK;
}

}  // namespace pa
