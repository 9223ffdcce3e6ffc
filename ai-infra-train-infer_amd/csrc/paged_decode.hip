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
//  * Wave w of W walks tiles w, w+W, ... of 16 tokens (fp16/bf16: two row loads) or 32 tokens
//    (fp8: four row loads).  The loads of the next tile and the table entries of the one after
//    are issued before the current tile is consumed, which keeps 8 KiB per wave in flight.
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

template <int KV, int D, int HPW = 1>
struct Geo {
  static constexpr int ES = (KV == KV_FP8) ? 1 : 2;  // bytes per cache element
  static constexpr int LPR = 8;                       // lanes per token row
  static constexpr int EPL = D / LPR;                 // elements per lane per token
  static constexpr int BPL = EPL * ES;                // bytes per lane per token
  static constexpr int LB = BPL >= 16 ? 16 : BPL;     // bytes per load instruction
  static constexpr int NLD = BPL / LB;                // loads per lane per token
  static constexpr int WPT = BPL / 4;                 // dwords per lane per token
  static constexpr int EPC = LB / ES;                 // elements per load
  // row loads (8 tokens each) per register tile: sized so a tile is 32 dwords of K + 32 of V
  // per lane at most, i.e. 16 tokens of fp16 or 32 tokens of fp8 at head_dim 128
  static constexpr int RL = (16 / WPT) < 4 ? (16 / WPT) : 4;
  static constexpr int RPL = 8 / HPW;                 // token rows per row load
  static constexpr int TILE = RPL * RL;               // tokens per tile
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

template <int KV, int D, int HPW>
struct Tile {
  using G = Geo<KV, D, HPW>;
  uint32_t k[G::RL][G::WPT];
  uint32_t v[G::RL][G::WPT];
  float ks[G::RL];
  float vs[G::RL];
};

// HPW = KV heads per wavefront.  With HPW == 2 the 8-lane row groups alternate between two
// adjacent KV heads, so 16 consecutive lanes read 2 x (head_dim * element size) contiguous
// bytes: rows of 128 bytes or less (fp8 at head_dim 128, anything at head_dim 64) are then
// fetched as 256-byte pieces, which HBM serves about 10% faster than lone 128-byte lines; wider
// rows gain from it when it lets the launch run as fewer, longer-lived workgroups (the launch
// code decides).
template <int KV, int D, int GC, int W, int HPW>
__global__ __launch_bounds__(W * 64) void paged_decode_kernel(const DecodeParams p) {
  using G = Geo<KV, D, HPW>;
  using TileT = Tile<KV, D, HPW>;
  constexpr int EPL = G::EPL;
  constexpr int RL = G::RL;
  constexpr int RPL = G::RPL;
  constexpr int TILE = G::TILE;
  constexpr int GCW = GC * HPW;  // query heads per workgroup
  constexpr int NG = W * 4;      // partial outputs per head that reach LDS
  constexpr float NEG_INF = -INFINITY;

  __shared__ float red[NG][GCW * D];
  __shared__ float sm[GCW][W];
  __shared__ float sl[GCW][W];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 3;        // row group 0..7
  const int j = lane & 7;         // position inside the row
  const int hs = g % HPW;         // which of the wave's KV heads this row group reads
  const int tr = g / HPW;         // token row inside a row load
  // blockIdx.x (fastest) walks the head groups, so the workgroups that share a token row are
  // dispatched together and land on different XCDs: each L2 fetches only its own head's bytes.
  const int b = blockIdx.z;
  const int part = blockIdx.y;
  const int h0 = blockIdx.x * GCW;                                   // first query head of the workgroup
  const int kvh = h0 / (p.num_q_heads / p.num_kv_heads) + hs;       // this lane's KV head
  const int hq = h0 + hs * GC;                                       // this lane's first query head

  const int ctx = p.context_lens[b];
  if (ctx <= 0) {
    // padded batch row: the output row is zero; the merge kernel does the same when partitioned
    if (p.direct_out && part == 0) {
      for (int o = threadIdx.x; o < GCW * D; o += W * 64)
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
  // the dtype switch sits outside the loops: inside, it would put a branch and a wait between
  // loads that are meant to be in flight together
  auto load_q = [&](auto dt_tag) __attribute__((always_inline)) {
#pragma unroll
    for (int h = 0; h < GC; ++h) {
      const int64_t base = b * p.q_stride + (int64_t)(hq + h) * D;
#pragma unroll
      for (int k = 0; k < EPL; k += 8) {
        float x[8];
        load8_as_f32(p.q, base + G::dim_of(k, j), decltype(dt_tag)::value, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[h][k + e] = x[e] * p.scale_log2e;
      }
    }
  };
  if (p.q_dtype == PA_DTYPE_F16) load_q(std::integral_constant<int, PA_DTYPE_F16>{});
  else if (p.q_dtype == PA_DTYPE_BF16) load_q(std::integral_constant<int, PA_DTYPE_BF16>{});
  else load_q(std::integral_constant<int, PA_DTYPE_F32>{});

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
  const uint32_t lane_off = (uint32_t)((tr * p.num_kv_heads + kvh) * D * G::ES + j * G::LB);
  const int32_t* bt_row = p.block_tables + b * p.bt_stride;
  // never index past the table row, even if a context length is larger than the row holds
  const int last_blk = min((end - 1) >> p.bs_log2, max((int)p.bt_stride - 1, 0));
  const int nfull = (end - begin) / TILE;        // whole tiles of the partition
  const bool has_tail = ((end - begin) % TILE) != 0;

  // physical block ids of the two row loads of a tile (wave-uniform scalar loads)
  auto load_ids = [&](int tile, int (&ids)[RL]) {
#pragma unroll
    for (int r = 0; r < RL; ++r) {
      const int tok = begin + tile * TILE + r * RPL;
      const int blk = min(tok >> p.bs_log2, last_blk);
      ids[r] = bt_row[blk];
    }
  };
  // start the K/V (and scale) loads of a tile; ids are clamped to the pool so that a corrupt
  // table can never fault
  auto issue = [&](TileT& t, int tile, const int (&ids)[RL]) {
#pragma unroll
    for (int r = 0; r < RL; ++r) {
      const int tok = begin + tile * TILE + r * RPL;
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
        t.ks[r] = p.k_scale[slot + tr];
        t.vs[r] = p.v_scale[slot + tr];
      }
    }
  };

  auto consume = [&](TileT& t, int tile, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    float s[RL][GC];
    bool valid[RL];
#pragma unroll
    for (int r = 0; r < RL; ++r) valid[r] = true;
#pragma unroll
    for (int r = 0; r < RL; ++r) {
      if constexpr (MASKED) valid[r] = (begin + tile * TILE + r * RPL + tr) < end;
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
      float mt = s[0][h];
#pragma unroll
      for (int r = 1; r < RL; ++r) mt = fmaxf(mt, s[r][h]);
      m_new[h] = fmaxf(m[h], mt);
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
    for (int r = 0; r < RL; ++r) {
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
    TileT ta, tb;
    int ids_a[RL], ids_b[RL];
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
    TileT tt;
    int ids_t[RL];
    load_ids(nfull, ids_t);
    issue(tt, nfull, ids_t);
    consume(tt, nfull, std::true_type{});
  }

  // ---- merge the row groups: common max, then plain sums (DPP, shuffles, LDS) ----------------
  // All 8 lanes of a row group hold the same m and l.  Groups of the same KV head differ in
  // lane bits 3..5 (HPW == 1) or 4..5 (HPW == 2, where bit 3 selects the head).
  const bool writer = (j == 0) && (tr == 0);  // lane 0, plus lane 8 when it owns the second head
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    float wm = m[h];
    if constexpr (HPW == 1) wm = fmaxf(wm, dpp_f32<0x128>(wm));  // row_ror:8 = lane ^ 8
    wm = fmaxf(wm, __shfl_xor(wm, 16));
    wm = fmaxf(wm, __shfl_xor(wm, 32));
    if (writer) sm[hs * GC + h][wave] = wm;
  }
  __syncthreads();
  float mx[GC];
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    float v = sm[hs * GC + h][0];
#pragma unroll
    for (int i = 1; i < W; ++i) v = fmaxf(v, sm[hs * GC + h][i]);
    mx[h] = v;  // finite: the partition holds at least one token
  }
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    const float w = __builtin_amdgcn_exp2f(m[h] - mx[h]);  // exp2(-inf) = 0 for idle groups
    float lw = l[h] * w;
    if constexpr (HPW == 1) lw += dpp_f32<0x128>(lw);
    lw += __shfl_xor(lw, 16);
    lw += __shfl_xor(lw, 32);
    if (writer) sl[hs * GC + h][wave] = lw;
#pragma unroll
    for (int k = 0; k < EPL; k += 4) {
      float o4[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float a = acc[h][k + e] * w;
        if constexpr (HPW == 1) a += dpp_f32<0x128>(a);  // pre-sum the two groups of a 16-lane row
        o4[e] = a;
      }
      if (HPW == 2 || (g & 1) == 0)
        *(float4*)&red[wave * 4 + (g >> 1)][(hs * GC + h) * D + G::dim_of(k, j)] =
            make_float4(o4[0], o4[1], o4[2], o4[3]);
    }
  }
  __syncthreads();
  for (int o = threadIdx.x; o < GCW * D; o += W * 64) {
    const int hh = o / D;  // query head relative to h0
    const int d = o - hh * D;
    float num = 0.0f, den = 0.0f;
#pragma unroll
    for (int i = 0; i < NG; ++i) num += red[i][o];
#pragma unroll
    for (int i = 0; i < W; ++i) den += sl[hh][i];
    const float res = num / den;
    if (p.direct_out) {
      store_from_f32(p.out, b * p.out_stride + (int64_t)(h0 + hh) * D + d, p.q_dtype, res);
    } else {
      const int64_t row = ((int64_t)b * p.num_q_heads + h0 + hh) * p.max_partitions + part;
      p.ws_out[row * D + d] = res;
      if (d == 0) {
        float mo = sm[hh][0];
#pragma unroll
        for (int i = 1; i < W; ++i) mo = fmaxf(mo, sm[hh][i]);
        p.ws_max[row] = mo * 0.6931471805599453f;  // back to natural-log units
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
static int g_decode_pair_heads = 1;   // 0 never, 1 automatic, 2 whenever the head layout allows

// CUs of the current device (per device, asked once).
static int compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

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

template <int KV, int D, int GC, int HPW>
static void launch_decode_w(const DecodeParams& p, dim3 grid, int waves, hipStream_t st) {
  switch (waves) {
    case 1: hipLaunchKernelGGL((paged_decode_kernel<KV, D, GC, 1, HPW>), grid, dim3(64), 0, st, p); break;
    case 2: hipLaunchKernelGGL((paged_decode_kernel<KV, D, GC, 2, HPW>), grid, dim3(128), 0, st, p); break;
    case 8: hipLaunchKernelGGL((paged_decode_kernel<KV, D, GC, 8, HPW>), grid, dim3(512), 0, st, p); break;
    default: hipLaunchKernelGGL((paged_decode_kernel<KV, D, GC, 4, HPW>), grid, dim3(256), 0, st, p); break;
  }
}

template <int KV, int D, int GC>
static void launch_decode_h(const DecodeParams& p, dim3 grid, int waves, int hpw, hipStream_t st) {
  if (hpw == 2) launch_decode_w<KV, D, GC, 2>(p, grid, waves, st);
  else launch_decode_w<KV, D, GC, 1>(p, grid, waves, st);
}

template <int KV>
static int launch_decode_kv(const DecodeParams& p, dim3 grid, int d, int gc, int waves, int hpw,
                            hipStream_t st) {
  if (d == 128 && gc == 2) launch_decode_h<KV, 128, 2>(p, grid, waves, hpw, st);
  else if (d == 128 && gc == 1) launch_decode_h<KV, 128, 1>(p, grid, waves, hpw, st);
  else if (d == 64 && gc == 2) launch_decode_h<KV, 64, 2>(p, grid, waves, hpw, st);
  else if (d == 64 && gc == 1) launch_decode_h<KV, 64, 1>(p, grid, waves, hpw, st);
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
  // Two adjacent KV heads per wave (each KV head's query group must be handled whole, so that
  // adjacent workgroup heads are adjacent KV heads) when halving the workgroups does not add a
  // round of them over the CUs: a CU streams at a fixed rate however many workgroups it hosts,
  // the launch takes as long as its busiest CU, and fewer, longer-lived workgroups stream better
  // (185 -> 178 us at batch 64 / ctx 4096, fp16; rows of 128 bytes or less gain another 10% from
  // being read as 256-byte pieces).  With a workgroup or less per CU pairing would only idle CUs.
  const bool can_pair = g == gc && num_kv_heads % 2 == 0;
  bool pair = false;
  if (can_pair && g_decode_pair_heads != 0) {
    const int64_t cus = compute_units();
    const int64_t wgs = (num_q_heads / gc) * max_partitions * batch;      // unpaired
    const int64_t rounds = (wgs + cus - 1) / cus, paired_rounds = (wgs + 2 * cus - 1) / (2 * cus);
    pair = g_decode_pair_heads == 2 || wgs >= 8 * cus || 2 * paired_rounds <= rounds;
  }
  const int hpw = pair ? 2 : 1;
  dim3 grid((unsigned)(num_q_heads / (gc * hpw)), (unsigned)max_partitions, (unsigned)batch);
  int rc;
  switch (kv) {
    case KV_F16: rc = launch_decode_kv<KV_F16>(p, grid, (int)head_dim, gc, g_decode_waves, hpw, st); break;
    case KV_BF16: rc = launch_decode_kv<KV_BF16>(p, grid, (int)head_dim, gc, g_decode_waves, hpw, st); break;
    default: rc = launch_decode_kv<KV_FP8>(p, grid, (int)head_dim, gc, g_decode_waves, hpw, st); break;
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

extern "C" int pa_set_decode_pair_heads(int mode) {
  if (mode < 0 || mode > 2) return fail(PA_ERR_BAD_ARG, "pa_set_decode_pair_heads: must be 0, 1 or 2");
  g_decode_pair_heads = mode;
  return PA_OK;
}
