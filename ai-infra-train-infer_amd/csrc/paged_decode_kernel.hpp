// Paged decode attention kernel for gfx950 (single pass and partitioned pass share it).
//
// Reference semantics: src/inference/attention.py:317-382 (gather through the block table,
// fp8 dequant as fp8/scale, GQA map h -> h/G, softmax(q.K^T*scale).V) and :519-589 (one
// partition: locally normalised output + log-sum-exp).
//
// The path is HBM-bound: every K and V byte of the context is read exactly once and used
// for a handful of FMAs, so the kernel is organised around the loads.
//
//  * One workgroup per (batch row, group of KV heads, partition).  All query heads that share a
//    KV head are served by that one workgroup, so a K/V row leaves HBM once whatever the GQA
//    ratio: GC (1, 2 or 4) query heads live in a wave's registers, and QS groups of waves take
//    QS x GC query heads over the same tokens (the second group's loads hit the CU's own L2).
//  * A token's K (or V) row for one KV head is head_dim elements = 8 lanes x EPL elements.
//    A wavefront therefore covers 8 (token, KV head) rows per load instruction, every load is
//    16 bytes per lane and the 8 lanes of a row read one full 128-byte line (fp8, or half a
//    256-byte fp16 row; the second half is the lane's second load).  No byte is fetched twice,
//    so there is nothing for LDS to reuse in the main loop; LDS only carries the final
//    cross-wave reduction.
//  * HPW (1, 2, 4 or 8) adjacent KV heads per wave: the 8 row groups of a load instruction are
//    8/HPW tokens x HPW heads, i.e. HPW x head_dim x element size contiguous bytes per token.
//    HBM serves wider pieces better (a whole fp8 token row of 8 heads is 1 KiB), at the price
//    of HPW times fewer workgroups.
//  * Wave w of a group's WQ waves walks tiles w, w+WQ, ...  The loads of the next tile and the
//    table entries of the one after are issued before the current tile is consumed.
//  * q.K partial dots are reduced over the 8 lanes of a row with three DPP adds; each row
//    group keeps its own running max / sum / output slice (no cross-lane traffic in the
//    loop) and the groups are merged once at the end through LDS.
//  * fp8: bytes -> fp32 with v_cvt_pk_f32_fp8 in registers; the per-token scale is applied
//    to the score (K) and to the probability (V) instead of to 128 elements each.
//  * K and V are read with non-temporal loads (they are used once; HBM streams 11-13 % faster that
//    way) unless a neighbouring row of the batch maps the same first block: see load_words and
//    decode_range_is_private.
#pragma once

#include "pa_common.hpp"
#include "pa_host.hpp"

#include <math.h>

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
  int table_width;
  int bs_log2;
  int num_blocks;
  int partition_size;
  int max_partitions;
  int direct_out;
  int inner;        // workgroups per (batch row, partition): KV head groups x slices of the query group
  int xcd_rows;     // 1: workgroup x serves (row, partition) unit (x / 8 / inner) * 8 + x % 8, see the kernel
  int batch;        // rows of the block table (a row's neighbours are looked at for shared blocks)
  float scale_log2e;
  // Shared prefixes (matrix kernel only; group_desc == nullptr: off).  Rows come in groups of
  // consecutive batch rows whose first `shared partitions` x partition_size tokens are the same
  // physical blocks: those partitions are computed once per group, by the first num_prefix_wgs
  // workgroups, for all the group's rows at once; the other workgroups take every row's own
  // partitions from row_skip[row] on.
  const int32_t* group_desc;   // [groups][4]: first row (or first entry of group_rows), rows, shared partitions, unused
  const int32_t* group_rows;   // batch rows of the groups, one run per group; nullptr: a group's rows are consecutive
  int group_rows_len;          // entries of group_rows
  const int32_t* row_skip;     // [batch]: leading partitions of the row that its group computes
  int num_groups;              // entries of group_desc
  int num_prefix_wgs;          // groups x prefix_parts x inner
  int prefix_parts;            // most shared partitions of any group
  int suffix_parts;            // most own partitions of any row
};

// How a launch is cut: all fields are template parameters of the kernel it selects.
struct DecodeShape {
  int head_dim;   // 64 or 128
  int gc;         // query heads per wave and KV head: 1, 2 or 4; 16 = the matrix kernel (up to 16 as one MFMA operand)
  int hpw;        // KV heads per wave: 1, 2, 4 or 8
  int qs;         // wave groups over the same tokens, each with its own gc query heads: 1, 2 or 4
  int waves;      // waves per workgroup (all groups together): 1, 2, 4 or 8
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
  // row loads (8 rows each) per register tile: sized so a tile is 32 dwords of K + 32 of V
  // per lane at most, i.e. 16 tokens of fp16 or 32 tokens of fp8 at head_dim 128 and HPW 1
  static constexpr int RL = (16 / WPT) < 4 ? (16 / WPT) : 4;
  static constexpr int RPL = 8 / HPW;                 // tokens per row load
  static constexpr int TILE = RPL * RL;               // tokens per tile
  static_assert(LB == 16 || LB == 8, "unsupported row geometry");
  // head-dim index of the lane's k-th element: loads are interleaved so that the 8 lanes of
  // a row cover LPR*LB contiguous bytes per load instruction.
  __device__ static constexpr int dim_of(int k, int j) {
    return (k / EPC) * (LPR * EPC) + j * EPC + (k % EPC);
  }
};

// Partial outputs per head that one wave hands to the cross-wave reduction.  A wave holds
// 8 / HPW of them (one per token row group); they are pre-summed inside the wave until the
// reduction buffer of the whole workgroup fits 32 KiB.
__host__ __device__ constexpr int decode_partials_per_wave(int W, int GC, int HPW, int D) {
  int pw = 8 / HPW;
  while (pw > 1 && W * pw * GC * HPW * D * 4 > 32768) pw /= 2;
  return pw;
}

// LDS bytes of a workgroup: the reduction buffer, then per head and wave a max and a sum.
__host__ __device__ constexpr int decode_lds_bytes(int W, int GC, int HPW, int QS, int D) {
  const int pw = decode_partials_per_wave(W, GC, HPW, D);
  return W * pw * GC * HPW * D * 4 + 2 * (GC * HPW * QS) * (W / QS) * 4;
}

// STREAM: a non-temporal load (the `nt` bit): the line is not kept in the L2 or the last-level cache
// for a later reader.  K and V of a private context are read once per launch, and read this way HBM
// streams 11-13 % faster (batch 64 x 4096 tokens: 178.9 -> 158.9 us on fp16, 99.7 -> 92.1 us on fp8).
// Blocks that other rows of the batch map as well are loaded normally, so that those rows hit.
template <int LB, bool STREAM>
__device__ __forceinline__ void load_words(const uint8_t* p, uint32_t* w) {
  typedef uint32_t u4_t __attribute__((ext_vector_type(4)));
  typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
  if constexpr (LB == 16) {
    u4_t v;
    if constexpr (STREAM) v = __builtin_nontemporal_load((const u4_t*)p);
    else v = *(const u4_t*)p;
    w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
  } else {
    u2_t v;
    if constexpr (STREAM) v = __builtin_nontemporal_load((const u2_t*)p);
    else v = *(const u2_t*)p;
    w[0] = v[0]; w[1] = v[1];
  }
}

// Whether a workgroup's K/V loads stream: yes, unless the first block of its token range is also
// the block at that place of the row before or after it in the batch.  Samples of one prompt and
// forks of a cached prefix sit next to each other and map the same physical blocks; their loads
// stay ordinary, so that the second reader of a block finds it in the L2.  A hint only: a table
// entry past a neighbour's context compares as whatever it holds.
__device__ __forceinline__ bool decode_range_is_private(const int32_t* bt_row, int64_t bt_stride, int b,
                                                        int batch, int first_blk) {
  const int own = bt_row[first_blk];
  const bool same_prev = b > 0 && bt_row[first_blk - bt_stride] == own;
  const bool same_next = b + 1 < batch && bt_row[first_blk + bt_stride] == own;
  return !(same_prev || same_next);
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

// Which token a lane holds in row load r of a tile.  16-bit caches: token r * RPL + tr (the 8 / HPW
// tokens of a row load are consecutive, so one table entry serves the whole load).  fp8 caches:
// token tr * RL + r - a lane's RL = 4 tokens are consecutive, so their per-token scales are one
// 16-byte load per lane and tile for K and one for V instead of a 4-byte load per row load (10
// vector memory instructions per fp8 tile instead of 16; the data loads are the same 128-byte
// rows either way).
template <int KV>
constexpr bool kLaneMajorTokens = (KV == KV_FP8);

template <int KV, int D, int HPW>
struct Tile {
  using G = Geo<KV, D, HPW>;
  uint32_t k[G::RL][G::WPT];
  uint32_t v[G::RL][G::WPT];
  float ks[G::RL];
  float vs[G::RL];
};

// Partitions of a row that hold tokens.
__device__ __forceinline__ int live_partitions(const DecodeParams& p, int row) {
  const int ctx = p.context_lens[row];
  return ctx <= 0 ? 0 : min((ctx + p.partition_size - 1) / p.partition_size, p.max_partitions);
}

// ... and how many of them are whole (the last one is not when the row ends inside it).
__device__ __forceinline__ int whole_partitions(const DecodeParams& p, int row) {
  const int ctx = p.context_lens[row];
  return ctx <= 0 ? 0 : min(ctx / p.partition_size, p.max_partitions);
}

// Lane l holds `mine`, a count for rows l * per_lane ... l * per_lane + per_lane - 1; count(row) gives
// one row's.  Finds the row that holds item u of the concatenation of all rows' items, and u's index
// inside that row; false when there are `total` <= u items.
template <typename Count>
__device__ __forceinline__ bool locate_item(int mine, int u, int lane, int per_lane, Count count, int& row, int& index,
                                            int& total) {
  int upto = mine;   // items of the rows of lanes 0 ... lane
  for (int d = 1; d < 64; d <<= 1) {
    const int t = __shfl_up(upto, d, 64);
    if (lane >= d) upto += t;
  }
  total = __shfl(upto, 63, 64);
  const unsigned long long past = __ballot(upto > u);
  if (past == 0) return false;
  const int owner = __ffsll(past) - 1;
  int base = __shfl(upto - mine, owner, 64);
  int r = owner * per_lane;
  // the owner's rows hold more than u - base items, so the walk ends inside them
  for (int i = 1; i < per_lane; ++i) {
    const int c = count(r);
    if (u < base + c) break;
    base += c;
    ++r;
  }
  row = r;
  index = u - base;
  return true;
}

// Work unit u of a partitioned launch -> (row, partition).  The grid is sized for batch x
// max_partitions units, but the units are the (row, partition) pairs that hold tokens: first the
// whole partitions, row by row, then the rows' last, shorter ones.  A ragged batch so packs its work
// into the first workgroups, the rest - one run at the end of the grid - leave at once (workgroups
// without work BETWEEN working ones are what costs: they hold the slots of a dispatch round that others
// wait for), and the short pieces come last, where they fill the gaps the long ones leave on the CUs.
// Every wave works the mapping out for itself, from the context lengths alone: lane l counts the
// partitions of rows l * k ... l * k + k - 1 (k = ceil(batch / 64)), a wave-wide running sum finds the
// lane whose rows hold unit u, a walk over that lane's rows the row.  False: u lies beyond the work of
// this launch.
__device__ __forceinline__ bool unit_to_row_partition(const DecodeParams& p, int u, int lane, int& row, int& part) {
  const int per_lane = (p.batch + 63) >> 6;
  const int first = lane * per_lane;
  int whole = 0, tails = 0;
  for (int i = 0; i < per_lane; ++i)
    if (first + i < p.batch) {
      const int w = whole_partitions(p, first + i);
      whole += w;
      tails += live_partitions(p, first + i) - w;
    }
  int total_whole;
  if (locate_item(whole, u, lane, per_lane, [&](int r) { return whole_partitions(p, r); }, row, part, total_whole))
    return true;
  int index, total_tails;
  if (!locate_item(tails, u - total_whole, lane, per_lane,
                   [&](int r) { return live_partitions(p, r) - whole_partitions(p, r); }, row, index, total_tails))
    return false;
  part = whole_partitions(p, row);     // the partition after the whole ones
  return true;
}

// W waves per workgroup in QS groups of WQ = W / QS.  Lane layout inside a wave: lane = 8 g + j,
// j the 16-byte piece of a row, g the row group; hs = g % HPW picks the KV head, tr = g / HPW
// the token of a row load.
// LOADS_ONLY (a measuring build, never instantiated by the library itself): every load of the
// launch is issued and every loaded word consumed, but the attention arithmetic is replaced by a
// checksum, so the launch lasts as long as the memory system needs for this access pattern.
template <int KV, int D, int GC, int W, int HPW, int QS, bool LOADS_ONLY = false>
__global__ __launch_bounds__(W * 64) void paged_decode_kernel(const DecodeParams p) {
  using G = Geo<KV, D, HPW>;
  using TileT = Tile<KV, D, HPW>;
  static_assert(QS == 1 || HPW == 1, "query-head groups of waves need one KV head per wave");
  static_assert(W % QS == 0, "waves must divide into the query-head groups");
  constexpr int EPL = G::EPL;
  constexpr int RL = G::RL;
  constexpr int RPL = G::RPL;
  constexpr int TILE = G::TILE;
  constexpr int WQ = W / QS;                 // waves that share the tokens of one query-head group
  constexpr int GCW = GC * HPW;              // query heads per wave
  constexpr int NH = GCW * QS;               // query heads per workgroup
  constexpr int RG = 8 / HPW;                // token row groups per wave (partials per head before pre-summing)
  constexpr int PW = decode_partials_per_wave(W, GC, HPW, D);
  constexpr int RED = RG / PW;               // row groups pre-summed into one partial
  constexpr int NG = WQ * PW;                // partials per head that reach LDS
  constexpr float NEG_INF = -INFINITY;

  extern __shared__ __align__(16) float lds[];
  float (*red)[GCW * D] = reinterpret_cast<float (*)[GCW * D]>(lds);          // [W * PW][GCW * D]
  float (*sm)[WQ] = reinterpret_cast<float (*)[WQ]>(lds + W * PW * GCW * D);  // [NH][WQ]
  float (*sl)[WQ] = sm + NH;                                                  // [NH][WQ]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int qgrp = wave / WQ;     // which GC query heads of the KV head this wave serves
  const int wv = wave % WQ;       // the wave's turn among the tiles
  const int g = lane >> 3;        // row group 0..7
  const int j = lane & 7;         // position inside the row
  const int hs = g % HPW;         // which of the wave's KV heads this row group reads
  const int tr = g / HPW;         // token inside a row load
  // Workgroups go to the 8 XCDs round robin by their index.  blockIdx.x walks the KV head groups
  // first, so the workgroups that share a token row are dispatched together and land on
  // different XCDs: each L2 fetches only its own heads' bytes (putting them on one XCD instead
  // measured 3% slower).  Then - only when one workgroup cannot hold a KV head's whole query
  // group - the slices of the query group.
  int in = blockIdx.x % p.inner;
  int u = blockIdx.x / p.inner;
  if (p.xcd_rows) {
    // fp8 caches: the workgroups of one (row, partition) on ONE XCD instead (workgroup x runs on XCD
    // x % 8): they all read the same per-token scales, and this way a scale line leaves HBM for one
    // L2 instead of four (batch 64 x 4096 tokens: 90.9 -> 89.9 us; the fp16 launch, which has no
    // scales to share, loses 4 % by it).
    const int x = blockIdx.x;
    const int slot = x >> 3;
    in = slot % p.inner;
    u = (slot / p.inner) * 8 + (x & 7);
  }
  int part = 0, b = u;
  if (p.max_partitions > 1 && !unit_to_row_partition(p, u, lane, b, part)) return;
  b = __builtin_amdgcn_readfirstlane(b);
  part = __builtin_amdgcn_readfirstlane(part);
  const int gq = p.num_q_heads / p.num_kv_heads;
  const int kv_groups = p.num_kv_heads / HPW;
  const int kvg = in % kv_groups;
  const int sub = in / kv_groups;
  const int h0 = kvg * HPW * gq + sub * (GC * QS);    // first query head of the workgroup
  const int kvh = kvg * HPW + hs;                     // this lane's KV head
  const int hl0 = (hs + qgrp) * GC;                   // this lane's first query head, relative to h0
  const int hq = h0 + hl0;

  const int ctx = p.context_lens[b];
  if (ctx <= 0) {
    // padded batch row: the output row is zero; the merge kernel does the same when partitioned
    if (p.direct_out && part == 0) {
      for (int o = threadIdx.x; o < NH * D; o += W * 64)
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
  constexpr bool LM = kLaneMajorTokens<KV>;
  // lane-major tiles: which of the tile's RL table entries (one per RPL tokens) covers this
  // lane's tokens tr * RL ... tr * RL + RL - 1
  int id_mask[RL];
#pragma unroll
  for (int r = 0; r < RL; ++r) id_mask[r] = (LM && (tr * RL) / RPL == r) ? -1 : 0;
  // byte offset of the lane's piece from the first token of its row load (row-major tiles: tr
  // tokens further on) or of its own token group (lane-major tiles)
  const uint32_t lane_off = (uint32_t)(((LM ? 0 : tr) * p.num_kv_heads + kvh) * D * G::ES + j * G::LB);
  const int32_t* bt_row = p.block_tables + b * p.bt_stride;
  // never index past the table row, even if a context length is larger than the row holds
  const int last_blk = min((end - 1) >> p.bs_log2, max(p.table_width - 1, 0));
  const int nfull = (end - begin) / TILE;        // whole tiles of the partition
  const bool has_tail = ((end - begin) % TILE) != 0;

  // physical block ids of the row loads of a tile (wave-uniform scalar loads)
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
  auto issue_as = [&](auto stream_tag, TileT& t, int tile, const int (&ids)[RL]) __attribute__((always_inline)) {
    constexpr bool STREAM = decltype(stream_tag)::value;
    if constexpr (LM) {
      static_assert(!LM || RL == 4, "lane-major tiles load four scales at once");
      // the table entry of this lane's four tokens: one of the tile's RL wave-uniform entries
      // (picked with per-lane bit masks: written as selects over the array, the compiler turns
      // the chain into an indexed read of a copy of `ids` in scratch memory)
      int id = 0;
#pragma unroll
      for (int r = 0; r < RL; ++r) id |= ids[r] & id_mask[r];
      const uint32_t phys = (uint32_t)min(max(id, 0), p.num_blocks - 1);
      const uint32_t off = (uint32_t)((begin + tile * TILE + tr * RL) & bs_mask);
      const uint64_t base = (uint64_t)phys * block_bytes + off * token_bytes + lane_off;
      const uint8_t* kp = p.k_cache + base;
      const uint8_t* vp = p.v_cache + base;
#pragma unroll
      for (int r = 0; r < RL; ++r) {
#pragma unroll
        for (int c = 0; c < G::NLD; ++c) {
          load_words<G::LB, STREAM>(kp + (r * token_bytes + c * G::LPR * G::LB), &t.k[r][c * (G::LB / 4)]);
          load_words<G::LB, STREAM>(vp + (r * token_bytes + c * G::LPR * G::LB), &t.v[r][c * (G::LB / 4)]);
        }
      }
      const uint64_t slot = ((uint64_t)phys << p.bs_log2) + off;
      const float4 k4 = *(const float4*)(p.k_scale + slot);
      const float4 v4 = *(const float4*)(p.v_scale + slot);
      t.ks[0] = k4.x; t.ks[1] = k4.y; t.ks[2] = k4.z; t.ks[3] = k4.w;
      t.vs[0] = v4.x; t.vs[1] = v4.y; t.vs[2] = v4.z; t.vs[3] = v4.w;
    } else {
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
          load_words<G::LB, STREAM>(kp + (lane_off + c * G::LPR * G::LB), &t.k[r][c * (G::LB / 4)]);
          load_words<G::LB, STREAM>(vp + (lane_off + c * G::LPR * G::LB), &t.v[r][c * (G::LB / 4)]);
        }
      }
    }
  };

  auto consume = [&](TileT& t, int tile, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    if constexpr (LOADS_ONLY) {
      uint32_t x = 0;
#pragma unroll
      for (int r = 0; r < RL; ++r) {
#pragma unroll
        for (int i = 0; i < G::WPT; ++i) x ^= t.k[r][i] ^ t.v[r][i];
        if constexpr (KV == KV_FP8) x ^= __float_as_uint(t.ks[r]) ^ __float_as_uint(t.vs[r]);
      }
      acc[0][0] += __uint_as_float(x & 0x3fffffffu);
      l[0] = 1.0f;
      m[0] = 0.0f;
    } else {
    float s[RL][GC];
    bool valid[RL];
#pragma unroll
    for (int r = 0; r < RL; ++r) valid[r] = true;
#pragma unroll
    for (int r = 0; r < RL; ++r) {
      if constexpr (MASKED) valid[r] = (begin + tile * TILE + (LM ? tr * RL + r : r * RPL + tr)) < end;
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
    }
  };

  // ---- main loop over this wave's whole tiles: wv, wv+WQ, ... < nfull ---------------------------
  // Two register tiles alternate between "in flight" and "being consumed"; the table entries
  // of a tile are fetched one step before its loads are issued.  The loop exists twice, with
  // streaming and with ordinary loads: chosen once per workgroup, so that each copy stays the
  // straight-line code the load / consume interleaving needs (a choice per tile cost 25 %).
  const int n_mine = nfull > wv ? (nfull - wv + WQ - 1) / WQ : 0;
  auto tile_of = [&](int i) { return wv + i * WQ; };
  auto run_tiles = [&](auto stream_tag) __attribute__((always_inline)) {
    auto issue = [&](TileT& t, int tile, const int (&ids)[RL]) __attribute__((always_inline)) {
      issue_as(stream_tag, t, tile, ids);
    };
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
    // ---- the partial last tile, masked, by the wave whose turn it is ------------------------------
    if (has_tail && (nfull % WQ) == wv) {
      TileT tt;
      int ids_t[RL];
      load_ids(nfull, ids_t);
      issue(tt, nfull, ids_t);
      consume(tt, nfull, std::true_type{});
    }
  };
  if (decode_range_is_private(bt_row, p.bt_stride, b, p.batch, min(begin >> p.bs_log2, last_blk)))
    run_tiles(std::true_type{});
  else
    run_tiles(std::false_type{});

  // ---- merge the row groups: common max, then plain sums (DPP, shuffles, LDS) ----------------
  // All 8 lanes of a row group hold the same m and l.  The RG row groups of one KV head differ in
  // the lane bits above those that select the head: bits 3..5 (HPW 1), 4..5 (HPW 2), 5 (HPW 4).
  const bool writer = (j == 0) && (tr == 0);  // one lane per KV head of the wave
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    float wm = m[h];
    if constexpr (HPW == 1) wm = fmaxf(wm, dpp_f32<0x128>(wm));  // row_ror:8 = lane ^ 8
    if constexpr (HPW <= 2) wm = fmaxf(wm, __shfl_xor(wm, 16));
    if constexpr (HPW <= 4) wm = fmaxf(wm, __shfl_xor(wm, 32));
    if (writer) sm[hl0 + h][wv] = wm;
  }
  __syncthreads();
  float mx[GC];
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    float v = sm[hl0 + h][0];
#pragma unroll
    for (int i = 1; i < WQ; ++i) v = fmaxf(v, sm[hl0 + h][i]);
    mx[h] = v;  // finite: the partition holds at least one token
  }
#pragma unroll
  for (int h = 0; h < GC; ++h) {
    const float w = __builtin_amdgcn_exp2f(m[h] - mx[h]);  // exp2(-inf) = 0 for idle groups
    float lw = l[h] * w;
    if constexpr (HPW == 1) lw += dpp_f32<0x128>(lw);
    if constexpr (HPW <= 2) lw += __shfl_xor(lw, 16);
    if constexpr (HPW <= 4) lw += __shfl_xor(lw, 32);
    if (writer) sl[hl0 + h][wv] = lw;
#pragma unroll
    for (int k = 0; k < EPL; k += 4) {
      float o4[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float a = acc[h][k + e] * w;
        // pre-sum RED row groups of the head: partner lanes differ in the lowest token bits
        if constexpr (RED >= 2) {
          if constexpr (HPW == 1) a += dpp_f32<0x128>(a);
          else a += __shfl_xor(a, 8 * HPW);
        }
        if constexpr (RED >= 4) a += __shfl_xor(a, 16 * HPW);
        if constexpr (RED >= 8) a += __shfl_xor(a, 32 * HPW);
        o4[e] = a;
      }
      if ((tr & (RED - 1)) == 0)
        *(float4*)&red[wave * PW + tr / RED][(hs * GC + h) * D + G::dim_of(k, j)] =
            make_float4(o4[0], o4[1], o4[2], o4[3]);
    }
  }
  __syncthreads();
  for (int o = threadIdx.x; o < NH * D; o += W * 64) {
    const int hh = o / D;           // query head relative to h0
    const int d = o - hh * D;
    const int qg = hh / GCW;        // the wave group that holds this head
    const int col = (hh - qg * GCW) * D + d;
    float num = 0.0f, den = 0.0f;
#pragma unroll
    for (int i = 0; i < NG; ++i) num += red[qg * NG + i][col];
#pragma unroll
    for (int i = 0; i < WQ; ++i) den += sl[hh][i];
    const float res = num / den;
    if (p.direct_out) {
      store_from_f32(p.out, b * p.out_stride + (int64_t)(h0 + hh) * D + d, p.q_dtype, res);
    } else {
      const int64_t row = ((int64_t)b * p.num_q_heads + h0 + hh) * p.max_partitions + part;
      p.ws_out[row * D + d] = res;
      if (d == 0) {
        float mo = sm[hh][0];
#pragma unroll
        for (int i = 1; i < WQ; ++i) mo = fmaxf(mo, sm[hh][i]);
        p.ws_max[row] = mo * 0.6931471805599453f;  // back to natural-log units
        p.ws_sum[row] = den;
      }
    }
  }
}

// ---- launch of one instantiation -------------------------------------------------------------

constexpr int kMaxDevices = 64;

template <int KV, int D, int GC, int W, int HPW, int QS, bool LOADS_ONLY = false>
static int launch_decode_one(const DecodeParams& p, dim3 grid, hipStream_t st) {
  constexpr int smem = decode_lds_bytes(W, GC, HPW, QS, D);
  auto kern = paged_decode_kernel<KV, D, GC, W, HPW, QS, LOADS_ONLY>;
  if constexpr (smem > 48 * 1024) {
    // above the default dynamic LDS limit: raise it once per instantiation and device
    static bool attr_set[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
      return fail(PA_ERR_LAUNCH, "pa_decode: cannot tell the current device");
    if (!__atomic_load_n(&attr_set[dev], __ATOMIC_ACQUIRE)) {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem) != hipSuccess)
        return fail(PA_ERR_LAUNCH, "pa_decode: cannot raise the dynamic LDS limit");
      __atomic_store_n(&attr_set[dev], true, __ATOMIC_RELEASE);
    }
  }
  hipLaunchKernelGGL(kern, grid, dim3(W * 64), smem, st, p);
  return PA_OK;
}

template <int KV, int D, int GC, int HPW>
static int launch_decode_waves(const DecodeParams& p, dim3 grid, int waves, hipStream_t st) {
  switch (waves) {
    case 1: return launch_decode_one<KV, D, GC, 1, HPW, 1>(p, grid, st);
    case 2: return launch_decode_one<KV, D, GC, 2, HPW, 1>(p, grid, st);
    case 4: return launch_decode_one<KV, D, GC, 4, HPW, 1>(p, grid, st);
    case 8:
      // four query heads per wave need more than the 256 registers a wave of an 8-wave workgroup gets
      if constexpr (GC < 4) return launch_decode_one<KV, D, GC, 8, HPW, 1>(p, grid, st);
      break;
  }
  return fail(PA_ERR_UNSUPPORTED, "pa_decode: unsupported waves per workgroup for this head layout");
}

// Instantiations with qs > 1: four query heads per wave in 4-wave workgroups (one wave per SIMD,
// ~280 registers), two per wave in 8-wave workgroups.
template <int KV, int D>
static int launch_decode_dim(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st) {
  if (s.qs > 1) {
    if (s.hpw == 1 && s.gc == 4 && s.waves == 4) {
      if (s.qs == 2) return launch_decode_one<KV, D, 4, 4, 1, 2>(p, grid, st);
      if (s.qs == 4) return launch_decode_one<KV, D, 4, 4, 1, 4>(p, grid, st);
    }
    if (s.hpw == 1 && s.gc == 2 && s.waves == 8) {
      if (s.qs == 2) return launch_decode_one<KV, D, 2, 8, 1, 2>(p, grid, st);
      if (s.qs == 4) return launch_decode_one<KV, D, 2, 8, 1, 4>(p, grid, st);
    }
    return fail(PA_ERR_UNSUPPORTED, "pa_decode: unsupported split of the query group over waves");
  }
  if (s.hpw == 1) {
    if (s.gc == 4) return launch_decode_waves<KV, D, 4, 1>(p, grid, s.waves, st);
    if (s.gc == 2) return launch_decode_waves<KV, D, 2, 1>(p, grid, s.waves, st);
    if (s.gc == 1) return launch_decode_waves<KV, D, 1, 1>(p, grid, s.waves, st);
  } else if (s.hpw == 2) {
    if (s.gc == 2) return launch_decode_waves<KV, D, 2, 2>(p, grid, s.waves, st);
    if (s.gc == 1) return launch_decode_waves<KV, D, 1, 2>(p, grid, s.waves, st);
  } else if ((s.hpw == 4 || s.hpw == 8) && s.gc == 2 && (s.waves == 4 || s.waves == 8)) {
    if (s.hpw == 4) return s.waves == 4 ? launch_decode_one<KV, D, 2, 4, 4, 1>(p, grid, st)
                                        : launch_decode_one<KV, D, 2, 8, 4, 1>(p, grid, st);
    return s.waves == 4 ? launch_decode_one<KV, D, 2, 4, 8, 1>(p, grid, st)
                        : launch_decode_one<KV, D, 2, 8, 8, 1>(p, grid, st);
  }
  return fail(PA_ERR_UNSUPPORTED, "pa_decode: unsupported combination of heads per wave and waves");
}

template <int KV>
static int launch_decode_mfma(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st);

template <int KV>
static int launch_decode_kv(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st) {
  if (s.gc == 16) return launch_decode_mfma<KV>(p, grid, s, st);
  if (s.head_dim == 128) return launch_decode_dim<KV, 128>(p, grid, s, st);
  if (s.head_dim == 64) return launch_decode_dim<KV, 64>(p, grid, s, st);
  return fail(PA_ERR_UNSUPPORTED, "pa_decode: head_dim must be 64 or 128");
}

// One translation unit per cache element type (they compile in parallel).
int launch_decode_f16(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st);
int launch_decode_bf16(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st);
int launch_decode_fp8(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st);

}  // namespace pa
