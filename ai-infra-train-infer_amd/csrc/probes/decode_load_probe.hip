// The decode launch with its arithmetic taken out (pa_decode_load_probe): the vector decode kernel
// of the product, instantiated with its loads-only template flag, behind the same argument checks
// and launch shaping as pa_decode_partials.  Part of the measuring library libpa_probes.so; the
// product library holds no instantiation of the loads-only build.
#include "paged_decode_launch.hpp"
#include "pa_probes.h"

namespace pa {

template <int KV>
static int launch_loads_only(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st) {
  if (s.head_dim == 128 && s.qs == 1 && s.waves == 4) {
    if (s.gc == 2 && s.hpw == 1) return launch_decode_one<KV, 128, 2, 4, 1, 1, true>(p, grid, st);
    if (s.gc == 2 && s.hpw == 2) return launch_decode_one<KV, 128, 2, 4, 2, 1, true>(p, grid, st);
    if (s.gc == 1 && s.hpw == 1) return launch_decode_one<KV, 128, 1, 4, 1, 1, true>(p, grid, st);
    if (s.gc == 1 && s.hpw == 2) return launch_decode_one<KV, 128, 1, 4, 2, 1, true>(p, grid, st);
  }
  return fail(PA_ERR_UNSUPPORTED,
              "pa_decode_load_probe: built for head_dim 128, 4-wave workgroups, 1 or 2 query heads per KV head, "
              "1 or 2 KV heads per wave");
}

}  // namespace pa

using namespace pa;

extern "C" int pa_decode_load_probe(const void* q, int q_dtype, int64_t q_token_stride,
                                    const void* k_cache, const void* v_cache, const float* k_scale,
                                    const float* v_scale, int kv_dtype, const int32_t* block_tables,
                                    int64_t bt_stride, int64_t table_width, const int32_t* context_lens,
                                    int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                    int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                    int64_t partition_size, int64_t max_partitions, void* workspace,
                                    int64_t workspace_bytes, int waves_per_workgroup,
                                    int kv_heads_per_wave, int q_heads_per_wave, void* stream) {
  DecodePlan plan;
  int rc = plan_decode("pa_decode_load_probe", q, q_dtype, q_token_stride, k_cache, v_cache, k_scale, v_scale,
                       kv_dtype, block_tables, bt_stride, table_width, context_lens, nullptr, 0, batch,
                       num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, 1.0f, partition_size,
                       max_partitions, workspace, workspace_bytes, waves_per_workgroup, kv_heads_per_wave,
                       q_heads_per_wave, false, true, nullptr, &plan);
  if (rc != PA_OK || plan.empty) return rc;
  const dim3 grid(plan.grid);
  switch (plan.kv) {
    case KV_F16: rc = launch_loads_only<KV_F16>(plan.p, grid, plan.s, (hipStream_t)stream); break;
    case KV_BF16: rc = launch_loads_only<KV_BF16>(plan.p, grid, plan.s, (hipStream_t)stream); break;
    default: rc = launch_loads_only<KV_FP8>(plan.p, grid, plan.s, (hipStream_t)stream); break;
  }
  if (rc != PA_OK) return rc;
  return check_launch("pa_decode_load_probe");
}
