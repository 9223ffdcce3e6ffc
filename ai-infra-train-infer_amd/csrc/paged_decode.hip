// Paged decode attention for gfx950: single pass, partitioned pass and the merge reduction.
//
// Reference semantics: src/inference/attention.py:317-382 (gather through the block table,
// fp8 dequant as fp8/scale, GQA map h -> h/G, softmax(q.K^T*scale).V), :519-589 (one
// partition: locally normalised output + log-sum-exp) and :591-626 (merge).
//
// The path is HBM-bound: every K and V byte of the context is read exactly once and used
// for a handful of FMAs, so the kernel is organised around the loads.
//
//  * One workgroup per (batch row, group of GC query heads sharing a KV head, partition).
//    Both query heads of a GQA pair live in registers, so a K/V row is fetched once.
//  * A token's K (or V) row for one KV head is head_dim elements = 8 lanes x EPL elements.
//    A wavefront therefore covers 8 token rows per load instruction, every load is 16 bytes
//    per lane and the 8 lanes of a row read one full 128-byte line (fp8, or half a 256-byte
//    fp16 row; the second half is the lane's second load).  No byte is fetched twice, so
//    there is nothing for LDS to reuse in the main loop; LDS only carries the final
//    cross-wave reduction.
//  * Wave w of W walks tiles w, w+W, ... of 16 tokens (two row loads).  The loads of the next
//    tile and the table entries of the one after are issued before the current tile is
//    consumed, which keeps 8 KiB (fp16) per wave in flight.
//  * q.K partial dots are reduced over the 8 lanes of a row with three DPP adds; each row
//    group keeps its own running max / sum / output slice (no cross-lane traffic in the
//    loop) and the groups are merged once at the end through LDS.
//  * fp8: bytes -> fp32 with v_cvt_pk_f32_fp8 in registers; the per-token scale is applied
//    to the score (K) and to the probability (V) instead of to 128 elements each.
#include "pa_common.hpp"
#include "pa_host.hpp"

#include <math.h>
#include <stdio.h>

#include <type_traits>

namespace pa {

struct DecodeParams {
  const void* q;
  int64_t q_stride;
  const uint8_t* k_cache;
  const uint8_t* v_cache;
  const float* k_scale;
  const float* v_scale;
  const int32_t* block_tables;
  int64_t bt_stride;
  const int32_t* context_lens;
  void* out;
  int64_t out_stride;
  float* ws_max;
  float* ws_sum;
  float* ws_out;
  int q_dtype;
  int num_q_heads;
  int num_kv_heads;
  int bs_log2;
  int num_blocks;
  int partition_size;
  int max_partitions;
  int direct_out;
  float scale_log2e;
};

template <int KV, int D>
struct Geo {
  static constexpr int ES = (KV == KV_FP8) ? 1 : 2;  // bytes per cache element
  static constexpr int LPR = 8;                       // lanes per token row
  static constexpr int EPL = D / LPR;                 // elements per lane per token
  static constexpr int BPL = EPL * ES;                // bytes per lane per token
  static constexpr int LB = BPL >= 16 ? 16 : BPL;     // bytes per load instruction
  static constexpr int NLD = BPL / LB;                // loads per lane per token
  static constexpr int WPT = BPL / 4;                 // dwords per lane per token
  static constexpr int EPC = LB / ES;                 // elements per load
  static_assert(LB == 16 || LB == 8, "unsupported row geometry");
  // head-dim index of the lane's k-th element: loads are interleaved so that the 8 lanes of
  // a row cover LPR*LB contiguous bytes per load instruction.
  __device__ static constexpr int dim_of(int k, int j) {
    return (k / EPC) * (LPR * EPC) + j * EPC + (k % EPC);
  }
};

template <int LB>
__device__ __forceinline__ void load_words(const uint8_t* p, uint32_t* w) {
  if constexpr (LB == 16) {
    const uint4 v = *(const uint4*)p;
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
  } else {
    const uint2 v = *(const uint2*)p;
    w[0] = v.x; w[1] = v.y;
  }
}

// dwords of one token row slice -> fp32 values
template <int KV, int WPT, int EPL>
__device__ __forceinline__ void unpack(const uint32_t (&w)[WPT], float (&x)[EPL]) {
#pragma unroll
  for (int i = 0; i < WPT; ++i) {
    if constexpr (KV == KV_F16) {
      const half2_t h = __builtin_bit_cast(half2_t, w[i]);
      x[2 * i] = (float)h[0];
      x[2 * i + 1] = (float)h[1];
    } else if constexpr (KV == KV_BF16) {
      x[2 * i] = __uint_as_float(w[i] << 16);
      x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    } else {
      const float2_t lo = fp8x2_to_f32(w[i], false);
      const float2_t hi = fp8x2_to_f32(w[i], true);
      x[4 * i] = lo[0];
      x[4 * i + 1] = lo[1];
      x[4 * i + 2] = hi[0];
      x[4 * i + 3] = hi[1];
    }
  }
}

template <int KV, int D>
struct Tile {
  using G = Geo<KV, D>;
  uint32_t k[2][G::WPT];
  uint32_t v[2][G::WPT];
  float ks[2];
  float vs[2];
};

template <int KV, int D, int GC, int W>
__global__ __launch_bounds__(W * 64) void paged_decode_kernel(const DecodeParams p) {
  using G = Geo<KV, D>;
  constexpr int EPL = G::EPL;
  constexpr int NG = W * 4;  // partial outputs that reach LDS (row groups, pairwise pre-summed)
  constexpr float NEG_INF = -INFINITY;

  __shared__ float red[NG][GC * D];
  __shared__ float sm[GC][W];
  __shared__ float sl[GC][W];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 3;
  const int j = lane & 7;
  const int b = blockIdx.z;
  const int part = blockIdx.y;
  const int h0 = blockIdx.x * GC;
  const int kvh = h0 / (p.num_q_heads / p.num_kv_heads);

  const int ctx = p.context_lens[b];
  if (ctx <= 0) {
    // padded batch row: the output row is zero; the merge kernel does the same when partitioned
    if (p.direct_out && part == 0) {
      for (int o = threadIdx.x; o < GC * D; o += W * 64)
        store_from_f32(p.out, b * p.out_stride + (int64_t)h0 * D + o, p.q_dtype, 0.0f);
    }
    return;
  }
  int begin = 0, end = ctx;
  if (p.max_partitions > 1) {
    begin = part * p.partition_size;
    end = (part == p.max_partitions - 1) ? ctx : min(begin + p.partition_size, ctx);
  }
  if (begin >= end) return;

  // ---- query: GC heads x EPL elements per lane, pre-multiplied by scale*log2(e) -------------
  float qf[GC][EPL];
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    const int64_t base = b * p.q_stride + (int64_t)(h0 + h) * D;
#pragma unroll
    for (int k = 0; k < EPL; k += 8) {
      float x[8];
      load8_as_f32(p.q, base + G::dim_of(k, j), p.q_dtype, x);
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[h][k + e] = x[e] * p.scale_log2e;
    }
  }

  float m[GC], l[GC], acc[GC][EPL];
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    m[h] = NEG_INF;
    l[h] = 0.0f;
#pragma unroll
    for (int k = 0; k < EPL; ++k) acc[h][k] = 0.0f;
  }

  const int bs_mask = (1 << p.bs_log2) - 1;
  const uint32_t token_bytes = (uint32_t)(p.num_kv_heads * D * G::ES);
  const uint32_t block_bytes = token_bytes << p.bs_log2;
  const uint32_t lane_off = (uint32_t)((g * p.num_kv_heads + kvh) * D * G::ES + j * G::LB);
  const int32_t* bt_row = p.block_tables + b * p.bt_stride;
  const int last_blk = (end - 1) >> p.bs_log2;
  const int nfull = (end - begin) >> 4;          // whole 16-token tiles of the partition
  const bool has_tail = ((end - begin) & 15) != 0;

  // physical block ids of the two row loads of a tile (wave-uniform scalar loads)
  auto load_ids = [&](int tile, int (&ids)[2]) {
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int tok = begin + tile * 16 + r * 8;
      const int blk = min(tok >> p.bs_log2, last_blk);
      ids[r] = bt_row[blk];
    }
  };
  // start the K/V (and scale) loads of a tile; ids are clamped to the pool so that a corrupt
  // table can never fault
  auto issue = [&](Tile<KV, D>& t, int tile, const int (&ids)[2]) {
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int tok = begin + tile * 16 + r * 8;
      const uint32_t phys = (uint32_t)min(max(ids[r], 0), p.num_blocks - 1);
      const uint32_t off = (uint32_t)(tok & bs_mask);
      const uint64_t base = (uint64_t)phys * block_bytes + off * token_bytes;
      const uint8_t* kp = p.k_cache + base;
      const uint8_t* vp = p.v_cache + base;
#pragma unroll
      for (int c = 0; c < G::NLD; ++c) {
        load_words<G::LB>(kp + (lane_off + c * G::LPR * G::LB), &t.k[r][c * (G::LB / 4)]);
        load_words<G::LB>(vp + (lane_off + c * G::LPR * G::LB), &t.v[r][c * (G::LB / 4)]);
      }
      if constexpr (KV == KV_FP8) {
        const uint64_t slot = ((uint64_t)phys << p.bs_log2) + off;
        t.ks[r] = p.k_scale[slot + g];
        t.vs[r] = p.v_scale[slot + g];
      }
    }
  };

  auto consume = [&](Tile<KV, D>& t, int tile, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    float s[2][GC];
    bool valid[2] = {true, true};
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      if constexpr (MASKED) valid[r] = (begin + tile * 16 + r * 8 + g) < end;
      float kf[EPL];
      unpack<KV, G::WPT, EPL>(t.k[r], kf);
      float inv_ks = 1.0f;
      if constexpr (KV == KV_FP8) inv_ks = __builtin_amdgcn_rcpf(t.ks[r]);
#pragma unroll
      for (int h = 0; h < GC; ++h) {
        float d0 = 0.0f, d1 = 0.0f;
#pragma unroll
        for (int k = 0; k < EPL; k += 2) {
          d0 = fmaf(qf[h][k], kf[k], d0);
          d1 = fmaf(qf[h][k + 1], kf[k + 1], d1);
        }
        float sc = sum8(d0 + d1);
        if constexpr (KV == KV_FP8) sc *= inv_ks;
        if constexpr (MASKED) sc = valid[r] ? sc : NEG_INF;
        s[r][h] = sc;
      }
    }
    float m_new[GC];
    bool changed = false;
#pragma unroll
    for (int h = 0; h < GC; ++h) {
      m_new[h] = fmaxf(m[h], fmaxf(s[0][h], s[1][h]));
      changed |= m_new[h] > m[h];
    }
    if (__builtin_amdgcn_ballot_w64(changed) != 0) {
#pragma unroll
      for (int h = 0; h < GC; ++h) {
        const float ms = (MASKED && m_new[h] == NEG_INF) ? 0.0f : m_new[h];
        const float alpha = __builtin_amdgcn_exp2f(m[h] - ms);
        l[h] *= alpha;
#pragma unroll
        for (int k = 0; k < EPL; ++k) acc[h][k] *= alpha;
        m[h] = m_new[h];
      }
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      if constexpr (MASKED) {
        if (!valid[r]) {
#pragma unroll
          for (int i = 0; i < G::WPT; ++i) t.v[r][i] = 0u;
        }
      }
      float vf[EPL];
      unpack<KV, G::WPT, EPL>(t.v[r], vf);
      float inv_vs = 1.0f;
      if constexpr (KV == KV_FP8) inv_vs = __builtin_amdgcn_rcpf(t.vs[r]);
#pragma unroll
      for (int h = 0; h < GC; ++h) {
        const float ms = (MASKED && m[h] == NEG_INF) ? 0.0f : m[h];
        const float pr = __builtin_amdgcn_exp2f(s[r][h] - ms);
        l[h] += pr;
        float pv = pr;
        if constexpr (KV == KV_FP8) {
          pv = pr * inv_vs;
          if constexpr (MASKED) pv = valid[r] ? pv : 0.0f;
        }
#pragma unroll
        for (int k = 0; k < EPL; ++k) acc[h][k] = fmaf(pv, vf[k], acc[h][k]);
      }
    }
  };

  // ---- main loop over this wave's whole tiles: wave, wave+W, ... < nfull ------------------------
  // Two register tiles alternate between "in flight" and "being consumed"; the table entries
  // of a tile are fetched one step before its loads are issued.
  const int n_mine = nfull > wave ? (nfull - wave + W - 1) / W : 0;
  auto tile_of = [&](int i) { return wave + i * W; };
  if (n_mine > 0) {
    Tile<KV, D> ta, tb;
    int ids_a[2], ids_b[2];
    load_ids(tile_of(0), ids_a);
    issue(ta, tile_of(0), ids_a);
    if (n_mine > 1) load_ids(tile_of(1), ids_b);
    int i = 0;
    for (; i + 1 < n_mine; i += 2) {
      issue(tb, tile_of(i + 1), ids_b);
      const bool more = i + 2 < n_mine;
      if (more) load_ids(tile_of(i + 2), ids_a);
      consume(ta, tile_of(i), std::false_type{});
      if (more) {
        issue(ta, tile_of(i + 2), ids_a);
        if (i + 3 < n_mine) load_ids(tile_of(i + 3), ids_b);
      }
      consume(tb, tile_of(i + 1), std::false_type{});
    }
    if (i < n_mine) consume(ta, tile_of(i), std::false_type{});
  }
  // ---- the partial last tile, masked, by the wave whose turn it is --------------------------------
  if (has_tail && (nfull % W) == wave) {
    Tile<KV, D> tt;
    int ids_t[2];
    load_ids(nfull, ids_t);
    issue(tt, nfull, ids_t);
    consume(tt, nfull, std::true_type{});
  }

  // ---- merge the W*8 row groups: common max, then plain sums (DPP, shuffles, LDS) ------------
  // all 8 lanes of a row group hold the same m and l, so lanes 8 apart are the partners
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    float wm = fmaxf(m[h], dpp_f32<0x128>(m[h]));  // row_ror:8 = lane ^ 8 inside a 16-lane row
    wm = fmaxf(wm, __shfl_xor(wm, 16));
    wm = fmaxf(wm, __shfl_xor(wm, 32));
    if (lane == 0) sm[h][wave] = wm;
  }
  __syncthreads();
  float mx[GC];
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    float v = sm[h][0];
#pragma unroll
    for (int i = 1; i < W; ++i) v = fmaxf(v, sm[h][i]);
    mx[h] = v;  // finite: the partition holds at least one token
  }
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    const float w = __builtin_amdgcn_exp2f(m[h] - mx[h]);  // exp2(-inf) = 0 for idle groups
    float lw = l[h] * w;
    lw += dpp_f32<0x128>(lw);
    lw += __shfl_xor(lw, 16);
    lw += __shfl_xor(lw, 32);
    if (lane == 0) sl[h][wave] = lw;
#pragma unroll
    for (int k = 0; k < EPL; k += 4) {
      float o4[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float a = acc[h][k + e] * w;
        o4[e] = a + dpp_f32<0x128>(a);
      }
      if ((g & 1) == 0)
        *(float4*)&red[wave * 4 + (g >> 1)][h * D + G::dim_of(k, j)] =
            make_float4(o4[0], o4[1], o4[2], o4[3]);
    }
  }
  __syncthreads();
  for (int o = threadIdx.x; o < GC * D; o += W * 64) {
    const int h = o / D;
    const int d = o - h * D;
    float num = 0.0f, den = 0.0f;
#pragma unroll
    for (int i = 0; i < NG; ++i) num += red[i][o];
#pragma unroll
    for (int i = 0; i < W; ++i) den += sl[h][i];
    const float res = num / den;
    if (p.direct_out) {
      store_from_f32(p.out, b * p.out_stride + (int64_t)(h0 + h) * D + d, p.q_dtype, res);
    } else {
      const int64_t row = ((int64_t)b * p.num_q_heads + h0 + h) * p.max_partitions + part;
      p.ws_out[row * D + d] = res;
      if (d == 0) {
        p.ws_max[row] = mx[h] * 0.6931471805599453f;  // back to natural-log units
        p.ws_sum[row] = den;
      }
    }
  }
}

// out = sum_p w_p out_p / sum_p w_p, w_p = sum_p * exp(max_p - max); one workgroup per
// (query head, batch row), one thread per head-dim element.
__global__ void merge_partitions_kernel(const float* __restrict__ ws_max,
                                        const float* __restrict__ ws_sum,
                                        const float* __restrict__ ws_out,
                                        const int32_t* __restrict__ context_lens, void* out,
                                        int out_dtype, int64_t out_stride, int num_q_heads,
                                        int head_dim, int partition_size, int max_partitions) {
  const int h = blockIdx.x;
  const int b = blockIdx.y;
  const int d = threadIdx.x;
  const int ctx = context_lens[b];
  const int64_t o = b * out_stride + (int64_t)h * head_dim + d;
  if (ctx <= 0) {
    store_from_f32(out, o, out_dtype, 0.0f);
    return;
  }
  const int np = min((ctx + partition_size - 1) / partition_size, max_partitions);
  const int64_t row0 = ((int64_t)b * num_q_heads + h) * max_partitions;
  float mx = -INFINITY;
  for (int q = 0; q < np; ++q) mx = fmaxf(mx, ws_max[row0 + q]);
  float num = 0.0f, den = 0.0f;
  for (int q = 0; q < np; ++q) {
    const float w = ws_sum[row0 + q] * __expf(ws_max[row0 + q] - mx);
    den += w;
    num = fmaf(w, ws_out[(row0 + q) * head_dim + d], num);
  }
  store_from_f32(out, o, out_dtype, num / den);
}

static int g_decode_waves = 4;

struct Workspace {
  float* mx;
  float* sum;
  float* out;
};

static int64_t ws_bytes(int64_t batch, int64_t hq, int64_t d, int64_t maxp) {
  if (maxp < 1) maxp = 1;
  const int64_t rows = batch * hq * maxp;
  // max and sum are padded to a 256-byte boundary so the partial outputs stay 16-byte aligned
  const int64_t scalars = ((rows * 4 + 255) / 256) * 256;
  return 2 * scalars + rows * d * 4;
}

static Workspace ws_split(void* ws, int64_t batch, int64_t hq, int64_t maxp) {
  const int64_t rows = batch * hq * maxp;
  const int64_t scalars = ((rows * 4 + 255) / 256) * 256;
  Workspace w;
  w.mx = (float*)ws;
  w.sum = (float*)((uint8_t*)ws + scalars);
  w.out = (float*)((uint8_t*)ws + 2 * scalars);
  return w;
}

template <int KV, int D, int GC>
static void launch_decode_w(const DecodeParams& p, dim3 grid, int waves, hipStream_t st) {
  switch (waves) {
    case 1: hipLaunchKernelGGL((paged_decode_kernel<KV, D, GC, 1>), grid, dim3(64), 0, st, p); break;
    case 2: hipLaunchKernelGGL((paged_decode_kernel<KV, D, GC, 2>), grid, dim3(128), 0, st, p); break;
    case 8: hipLaunchKernelGGL((paged_decode_kernel<KV, D, GC, 8>), grid, dim3(512), 0, st, p); break;
    default: hipLaunchKernelGGL((paged_decode_kernel<KV, D, GC, 4>), grid, dim3(256), 0, st, p); break;
  }
}

template <int KV>
static int launch_decode_kv(const DecodeParams& p, dim3 grid, int d, int gc, int waves,
                            hipStream_t st) {
  if (d == 128 && gc == 2) launch_decode_w<KV, 128, 2>(p, grid, waves, st);
  else if (d == 128 && gc == 1) launch_decode_w<KV, 128, 1>(p, grid, waves, st);
  else if (d == 64 && gc == 2) launch_decode_w<KV, 64, 2>(p, grid, waves, st);
  else if (d == 64 && gc == 1) launch_decode_w<KV, 64, 1>(p, grid, waves, st);
  else return fail(PA_ERR_UNSUPPORTED, "pa_decode: head_dim must be 64 or 128");
  return PA_OK;
}

static int ilog2_exact(int64_t v) {
  if (v <= 0 || (v & (v - 1)) != 0) return -1;
  int l = 0;
  while ((int64_t(1) << l) < v) ++l;
  return l;
}

// Shared argument checking + launch of the attention pass; `merge` adds the reduction.
static int decode_impl(const char* who, const void* q, int q_dtype, int64_t q_token_stride,
                       const void* k_cache, const void* v_cache, const float* k_scale,
                       const float* v_scale, int kv_dtype, const int32_t* block_tables,
                       int64_t bt_stride, const int32_t* context_lens, void* out,
                       int64_t out_token_stride, int64_t batch, int64_t num_q_heads,
                       int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                       int64_t num_blocks, float scale, int64_t partition_size,
                       int64_t max_partitions, void* workspace, int64_t workspace_bytes,
                       bool merge, void* stream) {
  char msg[256];
#define PA_FAIL(code, text)                         \
  do {                                              \
    snprintf(msg, sizeof(msg), "%s: %s", who, text); \
    return fail(code, msg);                         \
  } while (0)
  if (batch < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 ||
      num_blocks <= 0 || bt_stride < 0)
    PA_FAIL(PA_ERR_BAD_ARG, "negative or zero size");
  if (batch == 0) return PA_OK;
  if (!q || !k_cache || !v_cache || !block_tables || !context_lens)
    PA_FAIL(PA_ERR_BAD_ARG, "null pointer");
  if (merge && !out) PA_FAIL(PA_ERR_BAD_ARG, "null output");
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
  const bool direct = merge && max_partitions == 1;
  if (!direct) {
    if (max_partitions > 1 && (partition_size <= 0 || partition_size % 16 != 0))
      PA_FAIL(PA_ERR_UNSUPPORTED, "partition_size must be a positive multiple of 16");
    const int64_t need = ws_bytes(batch, num_q_heads, head_dim, max_partitions);
    if (!workspace || workspace_bytes < need) PA_FAIL(PA_ERR_WORKSPACE, "workspace missing or too small");
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
      PA_FAIL(PA_ERR_BAD_ARG, "workspace must be 256-byte aligned");
    if (partition_size > 0x7fffffff) PA_FAIL(PA_ERR_BAD_ARG, "partition_size too large");
  }
#undef PA_FAIL

  const int g = (int)(num_q_heads / num_kv_heads);
  const int gc = (g % 2 == 0) ? 2 : 1;

  DecodeParams p;
  p.q = q;
  p.q_stride = q_token_stride;
  p.k_cache = (const uint8_t*)k_cache;
  p.v_cache = (const uint8_t*)v_cache;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.block_tables = block_tables;
  p.bt_stride = bt_stride;
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

  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)(num_q_heads / gc), (unsigned)max_partitions, (unsigned)batch);
  int rc;
  switch (kv) {
    case KV_F16: rc = launch_decode_kv<KV_F16>(p, grid, (int)head_dim, gc, g_decode_waves, st); break;
    case KV_BF16: rc = launch_decode_kv<KV_BF16>(p, grid, (int)head_dim, gc, g_decode_waves, st); break;
    default: rc = launch_decode_kv<KV_FP8>(p, grid, (int)head_dim, gc, g_decode_waves, st); break;
  }
  if (rc != PA_OK) return rc;
  rc = check_launch(who);
  if (rc != PA_OK || direct || !merge) return rc;

  hipLaunchKernelGGL(merge_partitions_kernel, dim3((unsigned)num_q_heads, (unsigned)batch),
                     dim3((unsigned)head_dim), 0, st, p.ws_max, p.ws_sum, p.ws_out, context_lens,
                     out, q_dtype, out_token_stride, (int)num_q_heads, (int)head_dim,
                     (int)partition_size, (int)max_partitions);
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
                         const int32_t* context_lens, void* out, int64_t out_token_stride,
                         int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                         int64_t head_dim, int64_t block_size, int64_t num_blocks, float scale,
                         int64_t partition_size, int64_t max_partitions, void* workspace,
                         int64_t workspace_bytes, void* stream) {
  return decode_impl("pa_decode", q, q_dtype, q_token_stride, k_cache, v_cache, k_scale, v_scale,
                     kv_dtype, block_tables, bt_stride, context_lens, out, out_token_stride, batch,
                     num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, scale,
                     partition_size, max_partitions, workspace, workspace_bytes, true, stream);
}

extern "C" int pa_decode_partials(const void* q, int q_dtype, int64_t q_token_stride,
                                  const void* k_cache, const void* v_cache, const float* k_scale,
                                  const float* v_scale, int kv_dtype, const int32_t* block_tables,
                                  int64_t bt_stride, const int32_t* context_lens, int64_t batch,
                                  int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                  int64_t block_size, int64_t num_blocks, float scale,
                                  int64_t partition_size, int64_t max_partitions, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
  return decode_impl("pa_decode_partials", q, q_dtype, q_token_stride, k_cache, v_cache, k_scale,
                     v_scale, kv_dtype, block_tables, bt_stride, context_lens, nullptr, 0, batch,
                     num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, scale,
                     partition_size, max_partitions, workspace, workspace_bytes, false, stream);
}

extern "C" int pa_merge(const void* workspace, int64_t workspace_bytes, const int32_t* context_lens,
                        void* out, int out_dtype, int64_t out_token_stride, int64_t batch,
                        int64_t num_q_heads, int64_t head_dim, int64_t partition_size,
                        int64_t max_partitions, void* stream) {
  if (batch < 0 || num_q_heads <= 0 || head_dim <= 0 || max_partitions < 1 || partition_size <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_merge: bad size");
  if (batch == 0) return PA_OK;
  if (!workspace || !context_lens || !out) return fail(PA_ERR_BAD_ARG, "pa_merge: null pointer");
  if (head_dim > 1024) return fail(PA_ERR_UNSUPPORTED, "pa_merge: head_dim > 1024");
  if (out_dtype != PA_DTYPE_F16 && out_dtype != PA_DTYPE_BF16 && out_dtype != PA_DTYPE_F32)
    return fail(PA_ERR_UNSUPPORTED, "pa_merge: out_dtype must be f16, bf16 or f32");
  if (workspace_bytes < ws_bytes(batch, num_q_heads, head_dim, max_partitions))
    return fail(PA_ERR_WORKSPACE, "pa_merge: workspace too small");
  if (batch > 65535) return fail(PA_ERR_UNSUPPORTED, "pa_merge: batch too large");
  const Workspace w = ws_split(const_cast<void*>(workspace), batch, num_q_heads, max_partitions);
  hipLaunchKernelGGL(merge_partitions_kernel, dim3((unsigned)num_q_heads, (unsigned)batch),
                     dim3((unsigned)head_dim), 0, (hipStream_t)stream, w.mx, w.sum, w.out,
                     context_lens, out, out_dtype, out_token_stride, (int)num_q_heads,
                     (int)head_dim, (int)partition_size, (int)max_partitions);
  return check_launch("pa_merge");
}

extern "C" int pa_set_decode_waves(int waves) {
  if (waves != 1 && waves != 2 && waves != 4 && waves != 8)
    return fail(PA_ERR_BAD_ARG, "pa_set_decode_waves: must be 1, 2, 4 or 8");
  g_decode_waves = waves;
  return PA_OK;
}

extern "C" int pa_get_decode_waves(void) { return g_decode_waves; }
