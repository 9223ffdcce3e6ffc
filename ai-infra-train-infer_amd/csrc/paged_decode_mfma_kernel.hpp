// Paged decode attention for wide query groups (GQA ratios of 4 and more) on the matrix cores.
//
// Reference semantics: src/inference/attention.py:317-382 and :519-589, as for the kernel in
// paged_decode_kernel.hpp.  That kernel multiplies on the vector ALU, 2 x head_dim FMAs per lane
// row and query head: with 4 or 8 query heads behind every KV head the arithmetic, not the
// memory, sets the pace.  Here up to 16 query heads of one KV head form one MFMA operand, so the
// arithmetic per loaded byte no longer grows with the group.
//
//  * One workgroup per (batch row, HPW adjacent KV heads, partition[, slice of 16 query heads]);
//    wave w walks the 32-token tiles w, w + W, ... of the partition on its own: no barrier in the
//    loop.  HPW = 2: a wave reads the rows of two adjacent KV heads as one contiguous piece per
//    token (256 bytes of fp8 instead of 128) and multiplies one head after the other.
//  * Loads are those of the vector kernel: 16 bytes per lane, the 8 lanes of a token row read one
//    contiguous piece, one register tile (32 tokens of K and of V) in flight per wave;
//    non-temporal unless a neighbouring row maps the same blocks.
//  * A landed tile is written (16-bit caches as they are, bf16 and fp8 converted to fp16: K bytes of
//    an fp8 cache as they are - exact in fp16 - with 1 / k_scale of the tile's tokens beside the tile
//    in LDS and applied to the scores after the first product; V bytes times the power of two of
//    1 / v_scale, exact as well, the mantissa of 1 / v_scale going into the probabilities) to the
//    wave's own 2 x 32 x head_dim fp16 of LDS, and the next tile's loads are issued into the freed
//    registers before the products start.
//  * S^T = K . Q^T with v_mfma_f32_16x16x32_f16: A = 16 keys x 32 dims read back with
//    ds_read_b128, B = Q^T (16 head columns, zero beyond the group) kept in registers, pre-scaled
//    by scale*log2(e) and, for 16-bit caches, split into two fp16 parts (hi + lo, two products per
//    step); the accumulator starts at -m_ref so exp2 applies directly to the result.
//  * O^T += V^T . P^T: A = 16 dims x 32 keys through the LDS transpose read ds_read_b64_tr_b16,
//    B = P^T straight from the score registers (lane (head, g) holds keys 4g..4g+3 of both
//    16-key halves; the products label the contraction index accordingly).
//  * Shared prefixes (DecodeParams::group_desc): the columns of the operand can also be the query
//    heads of several batch rows, for partitions whose tokens those rows share as the same physical
//    blocks - read once for the group instead of once per row.
//  * The reference maximum m_ref is shared by the 4 lanes of a head column and only moves when a
//    tile's maximum outgrows it by more than 2^8; the waves' partial results are merged through
//    LDS at the end exactly as in the vector kernel.
#pragma once

#include "paged_decode_kernel.hpp"

namespace pa {

typedef _Float16 mhalf8_t __attribute__((ext_vector_type(8)));
typedef _Float16 mhalf4_t __attribute__((ext_vector_type(4)));
typedef __fp16 mfp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef float mfloat4_t __attribute__((ext_vector_type(4)));

constexpr int kMfmaTile = 32;    // tokens per tile
constexpr int kMfmaHeads = 16;   // query-head columns of the matrix operand

// 16-byte chunk c of LDS row r lives at chunk position c ^ lds_swz(r): 16 consecutive rows map one
// chunk index to 16 different positions (the A-operand reads of K), 4 consecutive rows differ in
// bits 2..3 (the 4-row patches of the transpose reads of V).
template <int CPR>
__device__ __forceinline__ constexpr int lds_swz(int row) {
  return (((row & 3) << 2) | ((row >> 2) & 3)) & (CPR - 1);
}

// K and V tile of one KV head
__host__ __device__ constexpr int decode_mfma_tile_bytes(int D) { return 2 * kMfmaTile * D * 2; }
// per wave: its tiles, then per token of the tile 1 / k_scale and the mantissa of 1 / v_scale (fp8 caches)
__host__ __device__ constexpr int decode_mfma_wave_bytes(int HPW, int D) {
  return HPW * decode_mfma_tile_bytes(D) + 2 * kMfmaTile * 4;
}
__host__ __device__ constexpr int decode_mfma_lds_bytes(int W, int HPW, int D) {
  return W * decode_mfma_wave_bytes(HPW, D) + 2 * HPW * kMfmaHeads * W * 4;
}

template <int KV, int D, int HPW>
struct MfmaTile {
  using G = Geo<KV, D, 1>;
  static constexpr int RL = 4 * HPW;     // row loads per tile: 8 / HPW tokens x HPW heads each
  uint32_t k[RL][G::WPT];
  uint32_t v[RL][G::WPT];
  float ks[RL];
  float vs[RL];
};

// 8 source elements (4 dwords of a 16-bit cache, 2 dwords of fp8) -> 8 fp16
template <int KV>
__device__ __forceinline__ mhalf8_t words_to_f16(const uint32_t* w) {
  mhalf8_t r;
  if constexpr (KV == KV_F16) {
    const uint32_t ww[4] = {w[0], w[1], w[2], w[3]};
    __builtin_memcpy(&r, ww, 16);
  } else if constexpr (KV == KV_BF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      r[2 * i] = (_Float16)__uint_as_float(w[i] << 16);
      r[2 * i + 1] = (_Float16)__uint_as_float(w[i] & 0xffff0000u);
    }
  } else {
    // the bytes as they are (exact in fp16); the token's scale is applied to the score and to the
    // probability after the products
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const half2_t lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[i], 1.0f, false);
      const half2_t hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[i], 1.0f, true);
      r[4 * i] = lo[0];
      r[4 * i + 1] = lo[1];
      r[4 * i + 2] = hi[0];
      r[4 * i + 3] = hi[1];
    }
  }
  return r;
}

// 8 fp8 bytes (2 dwords) times a power of two -> 8 fp16, exactly: v_cvt_scalef32_pk_f16_fp8 applies the
// exponent of its scale operand while it converts a pair.
__device__ __forceinline__ mhalf8_t fp8_words_to_f16_pow2(const uint32_t* w, float pow2) {
  mhalf8_t r;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const half2_t lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[i], pow2, false);
    const half2_t hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[i], pow2, true);
    r[4 * i] = lo[0];
    r[4 * i + 1] = lo[1];
    r[4 * i + 2] = hi[0];
    r[4 * i + 3] = hi[1];
  }
  return r;
}

template <int KV, int D, int W, int HPW>
__global__ __launch_bounds__(W * 64) void paged_decode_mfma_kernel(const DecodeParams p) {
  using G = Geo<KV, D, 1>;
  using TileT = MfmaTile<KV, D, HPW>;
  constexpr int TILE = kMfmaTile;
  constexpr int NHC = kMfmaHeads;
  constexpr int RPL = 8 / HPW;               // tokens per row load
  constexpr int RL = TileT::RL;              // row loads per tile
  constexpr int NSUB = RL / 4;               // lane-major tiles: groups of 4 row loads whose 4 tokens per lane are consecutive
  constexpr int EPS = RPL / 2;               // table entries (8 tokens each) per such group
  constexpr int CPR = D / 8;                 // 16-byte fp16 chunks per LDS row
  constexpr int ROWB = D * 2;                // bytes per LDS row
  constexpr int KSTEPS = D / 32;             // MFMA steps over head_dim in S
  constexpr int MT = D / 16;                 // 16-dim row tiles of O^T
  constexpr int CPL = G::EPC / 8;            // fp16 chunks per load instruction and lane (1, or 2 for fp8 at D 128)
  constexpr bool LM = kLaneMajorTokens<KV>;
  constexpr float NEG_INF = -INFINITY;
  constexpr int TILEB = decode_mfma_tile_bytes(D);

  extern __shared__ __align__(16) uint8_t lds_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int WAVEB = decode_mfma_wave_bytes(HPW, D);
  uint8_t* my_lds = lds_raw + wave * WAVEB;            // this wave's tiles: per KV head K, then V
  float* my_scales = reinterpret_cast<float*>(my_lds + HPW * TILEB);   // [2][TILE]: 1 / k_scale, mantissa of 1 / v_scale per token
  float (*red)[HPW * NHC * D] = reinterpret_cast<float (*)[HPW * NHC * D]>(lds_raw);   // [W][HPW * NHC * D], over the tiles
  float (*sm)[W] = reinterpret_cast<float (*)[W]>(lds_raw + W * WAVEB);                // [HPW * NHC][W]
  float (*sl)[W] = sm + HPW * NHC;                                                      // [HPW * NHC][W]

  const int g = lane >> 3;        // row group of the loads
  const int hs = g % HPW;         // which of the wave's KV heads this row group reads
  const int tr = g / HPW;         // token inside a row load
  const int j = lane & 7;         // 16-byte piece inside the row
  const int col = lane & 15;      // matrix layouts: head column / key row / dim row
  const int kg = lane >> 4;       // matrix layouts: group of 8 contraction indices, or of 4 result rows

  // ---- which rows, KV heads and tokens this workgroup takes ------------------------------------------------
  const int gq = p.num_q_heads / p.num_kv_heads;
  const int kv_groups = p.num_kv_heads / HPW;
  int b, part, in;
  int members = 1;          // batch rows served at once: > 1 only for the shared partitions of a group
  const int32_t* grows = nullptr;   // the group's rows when they are listed rather than consecutive
  if (p.group_desc) {
    // Descriptors come from device memory: everything read from them is brought into range before
    // it is used as an index, so that a corrupt descriptor gives wrong numbers, never a fault.
    // Workgroups that find nothing to do (a group with fewer shared partitions than the launch is sized
    // for, a padding group, a row with fewer partitions of its own) should sit together in the grid, not
    // between working ones: interleaved, 2048 of them cost the fourth benchmark configuration 32 us,
    // in one run at the end of a region next to nothing.  So both regions walk their partition index
    // last: all first partitions, then all second ones, ...
    int x = blockIdx.x;
    if (x < p.num_prefix_wgs) {
      in = x % p.inner;
      const int u = x / p.inner;
      part = u / p.num_groups;
      const int32_t* desc = p.group_desc + 4 * (u % p.num_groups);
      if (part >= desc[2]) return;
      members = min(desc[1], NHC / max(gq, 1));
      if (members < 1) return;
      if (p.group_rows) {
        const int first = desc[0];
        if (first < 0 || first + members > p.group_rows_len) return;
        grows = p.group_rows + first;
        b = grows[0];
      } else {
        b = desc[0];
        members = min(members, p.batch - b);
      }
      if (b < 0 || b >= p.batch || members < 1) return;
    } else {
      x -= p.num_prefix_wgs;
      in = x % p.inner;
      const int u = x / p.inner;
      b = u % p.batch;
      part = min(max(p.row_skip[b], 0), p.max_partitions) + u / p.batch;
      if (part >= p.max_partitions) return;
    }
  } else {
    in = blockIdx.x % p.inner;
    int u = blockIdx.x / p.inner;
    if (p.xcd_rows) {
      // fp8 caches: the workgroups of one (row, partition) on one XCD, where they share the row's scale
      // lines (the same mapping as in paged_decode_kernel)
      const int x = blockIdx.x;
      const int slot = x >> 3;
      in = slot % p.inner;
      u = (slot / p.inner) * 8 + (x & 7);
    }
    part = 0;
    b = u;
    if (p.max_partitions > 1) {
      if (!unit_to_row_partition(p, u, threadIdx.x & 63, b, part)) return;
      b = __builtin_amdgcn_readfirstlane(b);
      part = __builtin_amdgcn_readfirstlane(part);
    }
  }
  const int kvg = in % kv_groups;
  const int sub = in / kv_groups;
  const int kvh0 = kvg * HPW;                        // first KV head of the workgroup
  // Columns of the matrix operand.  One row: query heads sub * 16 ... of the KV head.  A group's
  // shared partition: column c = query head c % gq of the group's row c / gq (gq * members <= 16).
  const int cdiv = members > 1 ? gq : NHC + 1;
  const int nh = members > 1 ? members * gq : min(gq - sub * NHC, NHC);   // live columns per KV head
  auto first_head = [&](int hh) { return (kvh0 + hh) * gq + sub * NHC; };   // first query head behind KV head kvh0 + hh
  auto col_row = [&](int c) {
    const int i = c / cdiv;
    return grows ? min(max(grows[i], 0), p.batch - 1) : b + i;
  };
  auto col_head = [&](int hh, int c) { return first_head(hh) + c % cdiv; };

  const int ctx = p.context_lens[b];
  if (ctx <= 0) {
    if (p.direct_out && part == 0) {
      for (int o = threadIdx.x; o < HPW * nh * D; o += W * 64) {
        const int hh = o / (nh * D);
        store_from_f32(p.out, b * p.out_stride + (int64_t)first_head(hh) * D + (o - hh * nh * D), p.q_dtype, 0.0f);
      }
    }
    return;
  }
  int begin = 0, end = ctx;
  if (p.max_partitions > 1) {
    begin = part * p.partition_size;
    // the last partition takes whatever is left of the row's context; a shared one ends with the partition
    end = (part == p.max_partitions - 1 && members == 1) ? ctx : min(begin + p.partition_size, ctx);
  }
  if (begin >= end) return;

  // ---- Q^T as the B operand: lane (col, kg) holds dims 32c + 8kg .. +7 of head col, step c ----------
  // 16-bit caches: in two fp16 parts, q * scale * log2(e) = hi + lo to 22 bits.  The matrix pipe has
  // time to spare, and a single fp16 rounding of the query costs 2^-12 of the score, visible where
  // logits are large.  fp8 caches (tolerance 1e-2) take the one part.
  constexpr bool SPLIT_Q = KV != KV_FP8;
  mhalf8_t qreg[HPW][KSTEPS], qlo[SPLIT_Q ? HPW : 1][SPLIT_Q ? KSTEPS : 1];
  {
    const bool live = col < nh;
    auto load_q = [&](auto dt_tag) __attribute__((always_inline)) {
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {
        const int lc = live ? col : 0;
        const int64_t base = col_row(lc) * p.q_stride + (int64_t)col_head(hh, lc) * D + 8 * kg;
#pragma unroll
        for (int c = 0; c < KSTEPS; ++c) {
          float x[8];
          load8_as_f32(p.q, base + 32 * c, decltype(dt_tag)::value, x);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float qs = live ? x[e] * p.scale_log2e : 0.0f;
            const _Float16 hi = (_Float16)qs;
            qreg[hh][c][e] = hi;
            if constexpr (SPLIT_Q) qlo[hh][c][e] = (_Float16)(qs - (float)hi);
          }
        }
      }
    };
    if (p.q_dtype == PA_DTYPE_F16) load_q(std::integral_constant<int, PA_DTYPE_F16>{});
    else if (p.q_dtype == PA_DTYPE_BF16) load_q(std::integral_constant<int, PA_DTYPE_BF16>{});
    else load_q(std::integral_constant<int, PA_DTYPE_F32>{});
  }

  // ---- loads: as in the vector kernel ------------------------------------------------------------------
  // A row load covers 8 / HPW tokens x HPW heads.  16-bit caches: row load r holds tokens r * RPL + tr.
  // fp8 caches: a lane's 4 tokens of each group of 4 row loads are consecutive (token
  // 4 RPL (r / 4) + 4 tr + r % 4), so their scales are one 16-byte load.
  const int bs_mask = (1 << p.bs_log2) - 1;
  const uint32_t token_bytes = (uint32_t)(p.num_kv_heads * D * G::ES);
  const uint32_t block_bytes = token_bytes << p.bs_log2;
  auto token_of = [&](int r) { return LM ? (r / 4) * (4 * RPL) + tr * 4 + (r % 4) : r * RPL + tr; };
  int id_mask[EPS];     // lane-major tiles: which of a group's EPS table entries covers this lane's 4 tokens
#pragma unroll
  for (int x = 0; x < EPS; ++x) id_mask[x] = (LM && tr / 2 == x) ? -1 : 0;
  const uint32_t lane_off = (uint32_t)(((LM ? 0 : tr) * p.num_kv_heads + kvh0 + hs) * D * G::ES + j * G::LB);
  const int32_t* bt_row = p.block_tables + b * p.bt_stride;
  const int last_blk = min((end - 1) >> p.bs_log2, max(p.table_width - 1, 0));
  const int ntiles = (end - begin + TILE - 1) / TILE;

  // the tile's 4 table entries, one per 8 tokens (wave-uniform scalar loads)
  auto load_ids = [&](int tile, int (&ids)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int tok = begin + tile * TILE + x * 8;
      ids[x] = bt_row[min(tok >> p.bs_log2, last_blk)];
    }
  };
  auto issue_as = [&](auto stream_tag, TileT& t, int tile, const int (&ids)[4]) __attribute__((always_inline)) {
    constexpr bool STREAM = decltype(stream_tag)::value;
    if constexpr (LM) {
#pragma unroll
      for (int sb = 0; sb < NSUB; ++sb) {
        int id = 0;
#pragma unroll
        for (int x = 0; x < EPS; ++x) id |= ids[sb * EPS + x] & id_mask[x];
        const uint32_t phys = (uint32_t)min(max(id, 0), p.num_blocks - 1);
        const uint32_t off = (uint32_t)((begin + tile * TILE + sb * 4 * RPL + tr * 4) & bs_mask);
        const uint64_t base = (uint64_t)phys * block_bytes + off * token_bytes + lane_off;
        const uint8_t* kp = p.k_cache + base;
        const uint8_t* vp = p.v_cache + base;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
          for (int c = 0; c < G::NLD; ++c) {
            load_words<G::LB, STREAM>(kp + (r * token_bytes + c * G::LPR * G::LB), &t.k[4 * sb + r][c * (G::LB / 4)]);
            load_words<G::LB, STREAM>(vp + (r * token_bytes + c * G::LPR * G::LB), &t.v[4 * sb + r][c * (G::LB / 4)]);
          }
        }
        const uint64_t slot = ((uint64_t)phys << p.bs_log2) + off;
        const float4 k4 = *(const float4*)(p.k_scale + slot);
        const float4 v4 = *(const float4*)(p.v_scale + slot);
        t.ks[4 * sb] = k4.x; t.ks[4 * sb + 1] = k4.y; t.ks[4 * sb + 2] = k4.z; t.ks[4 * sb + 3] = k4.w;
        t.vs[4 * sb] = v4.x; t.vs[4 * sb + 1] = v4.y; t.vs[4 * sb + 2] = v4.z; t.vs[4 * sb + 3] = v4.w;
      }
    } else {
#pragma unroll
      for (int r = 0; r < RL; ++r) {
        const int tok = begin + tile * TILE + r * RPL;
        const uint32_t phys = (uint32_t)min(max(ids[(r * RPL) / 8], 0), p.num_blocks - 1);
        const uint64_t base = (uint64_t)phys * block_bytes + (uint32_t)(tok & bs_mask) * token_bytes;
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

  // ---- registers -> LDS: row = token of the tile, chunk = 8 head-dim elements ----------------------
  auto write_tile = [&](TileT& t, int tile, bool masked) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < RL; ++r) {
      const int tk = token_of(r);
      const bool valid = !masked || (begin + tile * TILE + tk) < end;
      // fp8: 1 / v_scale = m * 2^e with m in [1, 2).  The power of two goes into V here, on its way
      // into LDS (exact, and free: the conversion instruction applies it), the mantissa into the
      // probability before the second product, so that what is rounded to fp16 there is p * m, a number
      // in [0, 512].  (Folding all of 1 / v_scale - about amax / 448 - into the probability loses
      // every key whose p / v_scale falls below fp16's smallest subnormal while its p still counts in
      // the row sum: with small V behind an attention sink, tens of percent of the output.)
      float v_pow2 = 1.0f;
      if constexpr (KV == KV_FP8)
        v_pow2 = __uint_as_float(__float_as_uint(__builtin_amdgcn_rcpf(t.vs[r])) & 0xff800000u);
#pragma unroll
      for (int c = 0; c < G::NLD; ++c) {
#pragma unroll
        for (int x = 0; x < CPL; ++x) {
          const int chunk = (c * 8 + j) * CPL + x;
          const int wpc = (KV == KV_FP8) ? 2 : 4;   // dwords per 8 source elements
          mhalf8_t kf = words_to_f16<KV>(&t.k[r][c * (G::LB / 4) + x * wpc]);
          mhalf8_t vf;
          if constexpr (KV == KV_FP8) vf = fp8_words_to_f16_pow2(&t.v[r][c * (G::LB / 4) + x * wpc], v_pow2);
          else vf = words_to_f16<KV>(&t.v[r][c * (G::LB / 4) + x * wpc]);
          if (!valid) {
            // rows past the end: their scores are masked, and their V must not turn 0 * garbage into NaN
#pragma unroll
            for (int e = 0; e < 8; ++e) { kf[e] = (_Float16)0.0f; vf[e] = (_Float16)0.0f; }
          }
          uint8_t* dst = my_lds + hs * TILEB + tk * ROWB + ((chunk ^ lds_swz<CPR>(tk)) << 4);
          *(mhalf8_t*)dst = kf;
          *(mhalf8_t*)(dst + TILE * ROWB) = vf;
        }
      }
    }
    if constexpr (KV == KV_FP8) {
      // per token: 1 / k_scale (applied to the scores after the first product) and the mantissa of
      // 1 / v_scale (applied to the probabilities before the second); 0 for rows past the end (their
      // scores are masked and their V rows zero, and 0 * 0 stays 0).  The 8 lanes of a row group (and
      // both heads' groups) hold the same values and write the same words.
#pragma unroll
      for (int sb = 0; sb < NSUB; ++sb) {
        float ik[4], mv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const bool valid = !masked || (begin + tile * TILE + token_of(4 * sb + r)) < end;
          ik[r] = valid ? __builtin_amdgcn_rcpf(t.ks[4 * sb + r]) : 0.0f;
          const uint32_t bits = __float_as_uint(__builtin_amdgcn_rcpf(t.vs[4 * sb + r]));
          mv[r] = valid ? __uint_as_float((bits & 0x007fffffu) | 0x3f800000u) : 0.0f;
        }
        const int tok0 = token_of(4 * sb);
        *(float4*)&my_scales[tok0] = make_float4(ik[0], ik[1], ik[2], ik[3]);
        *(float4*)&my_scales[TILE + tok0] = make_float4(mv[0], mv[1], mv[2], mv[3]);
      }
    }
  };

  // ---- LDS read addresses ------------------------------------------------------------------------
  // (of the wave's first KV head; the second one's tiles lie TILEB further on)
  // K as A operand of S^T: key row col (+16 for the second half), dims 32c + 8kg .. +7
  const uint8_t* k_rd[KSTEPS];
#pragma unroll
  for (int c = 0; c < KSTEPS; ++c) k_rd[c] = my_lds + col * ROWB + (((4 * c + kg) ^ lds_swz<CPR>(col)) << 4);
  // V^T as A operand of O^T through the transpose read: within a block of 16 lanes (one kg), lane a
  // supplies the address of 4 dims of key 4kg + a/4 and receives those 4 keys of dim 16mt + a.
  const uint8_t* v_rd[MT];
  {
    const int key = 4 * kg + (col >> 2);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      v_rd[mt] = my_lds + TILE * ROWB + key * ROWB + (((2 * mt + ((col & 3) >> 1)) ^ lds_swz<CPR>(key)) << 4) + (col & 1) * 8;
  }

  float m_ref[HPW];       // per KV head; the same in the 4 lanes of a head column
  float l_run[HPW];       // this lane's share of the row sum
  mfloat4_t o[HPW][MT];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    m_ref[hh] = 0.0f;
    l_run[hh] = 0.0f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) o[hh][mt] = mfloat4_t{0.0f, 0.0f, 0.0f, 0.0f};
  }
  bool first = true;

  // All heads of the wave go through each phase together: the products of one phase are independent
  // chains (per head: two key halves x the two parts of the query), so the matrix pipe is never
  // waiting on a single accumulator, and the rare rescale is one branch for the whole wave.
  auto compute = [&](int tile, bool masked) __attribute__((always_inline)) {
    // ---- S^T: two 16-key halves; the hi-part accumulators start at -m_ref ----------------------------
    mfloat4_t s[HPW][2], s2[HPW][2];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      const float nr = KV == KV_FP8 ? 0.0f : -m_ref[hh];   // fp8: the scale comes first, the reference after it
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        s[hh][kb] = mfloat4_t{nr, nr, nr, nr};
        s2[hh][kb] = mfloat4_t{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
    // fp8: 1 / k_scale and the mantissa of 1 / v_scale of this lane's 8 keys (4kg .. 4kg+3 of both halves)
    float iks[2][4], mvs[2][4];
    if constexpr (KV == KV_FP8) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const float4 a = *(const float4*)&my_scales[16 * kb + 4 * kg];
        const float4 b2 = *(const float4*)&my_scales[TILE + 16 * kb + 4 * kg];
        iks[kb][0] = a.x; iks[kb][1] = a.y; iks[kb][2] = a.z; iks[kb][3] = a.w;
        mvs[kb][0] = b2.x; mvs[kb][1] = b2.y; mvs[kb][2] = b2.z; mvs[kb][3] = b2.w;
      }
    }
#pragma unroll
    for (int c = 0; c < KSTEPS; ++c)
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          const mhalf8_t a = *(const mhalf8_t*)(k_rd[c] + (hh * TILEB + kb * 16 * ROWB));
          s[hh][kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qreg[hh][c], s[hh][kb], 0, 0, 0);
          if constexpr (SPLIT_Q) s2[hh][kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qlo[hh][c], s2[hh][kb], 0, 0, 0);
        }
    const int lim = masked ? end - (begin + tile * TILE) : TILE;   // keys of the tile below this are real
    float mloc[HPW];
    bool want = first;
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float x;
          if constexpr (KV == KV_FP8) x = fmaf(s[hh][kb][e], iks[kb][e], -m_ref[hh]);
          else x = SPLIT_Q ? s[hh][kb][e] + s2[hh][kb][e] : s[hh][kb][e];
          s[hh][kb][e] = (16 * kb + 4 * kg + e) < lim ? x : NEG_INF;
        }
      float mx = s[hh][0][0];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 4; ++e) mx = fmaxf(mx, s[hh][kb][e]);
      mloc[hh] = mx;
      want |= mx > 8.0f;
    }
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(want) != 0, 0)) {
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {
        // the head column's maximum over its 4 lanes, then the same decision in all of them
        float hmax = fmaxf(mloc[hh], __shfl_xor(mloc[hh], 16));
        hmax = fmaxf(hmax, __shfl_xor(hmax, 32));
        const bool grow = first ? (hmax > NEG_INF) : (hmax > 8.0f);
        const float delta = grow ? hmax : 0.0f;
        const float alpha = first ? 1.0f : __builtin_amdgcn_exp2f(-delta);   // nothing accumulated before the first tile
        l_run[hh] *= alpha;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int e = 0; e < 4; ++e) o[hh][mt][e] *= alpha;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int e = 0; e < 4; ++e) s[hh][kb][e] -= delta;
        m_ref[hh] += delta;
      }
    }
    first = false;
    // ---- P^T as B operand: contraction index 8kg + e <-> key 4kg + e (e < 4), 16 + 4kg + e - 4 ------
    mhalf8_t pb[HPW];
    const half2_t one2 = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      float psum = 0.0f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          if constexpr (KV == KV_FP8) {
            // the row sum takes the probability, the product the probability times the mantissa of 1 / v_scale
            const float p0 = __builtin_amdgcn_exp2f(s[hh][kb][e]), p1 = __builtin_amdgcn_exp2f(s[hh][kb][e + 1]);
            psum += p0 + p1;
            pb[hh][4 * kb + e] = (_Float16)(p0 * mvs[kb][e]);
            pb[hh][4 * kb + e + 1] = (_Float16)(p1 * mvs[kb][e + 1]);
          } else {
            // the row sum adds exactly the fp16 values that the second product multiplies
            const half2_t h = {(_Float16)__builtin_amdgcn_exp2f(s[hh][kb][e]), (_Float16)__builtin_amdgcn_exp2f(s[hh][kb][e + 1])};
            psum = __builtin_amdgcn_fdot2(h, one2, psum, false);
            pb[hh][4 * kb + e] = h[0];
            pb[hh][4 * kb + e + 1] = h[1];
          }
        }
      l_run[hh] += psum;
    }
    // ---- O^T += V^T . P^T ------------------------------------------------------------------------
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {
        const mfp16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16((__attribute__((address_space(3))) mfp16x4_t*)(v_rd[mt] + hh * TILEB));
        const mfp16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16((__attribute__((address_space(3))) mfp16x4_t*)(v_rd[mt] + (hh * TILEB + 16 * ROWB)));
        const mhalf4_t l4 = __builtin_bit_cast(mhalf4_t, lo), h4 = __builtin_bit_cast(mhalf4_t, hi);
        const mhalf8_t a = {l4[0], l4[1], l4[2], l4[3], h4[0], h4[1], h4[2], h4[3]};
        o[hh][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pb[hh], o[hh][mt], 0, 0, 0);
      }
  };

  // ---- this wave's tiles: wave, wave + W, ... -------------------------------------------------------
  const int n_mine = ntiles > wave ? (ntiles - wave + W - 1) / W : 0;
  const bool has_tail = ((end - begin) % TILE) != 0;
  // The loop exists twice, with streaming and with ordinary loads (see load_words), chosen once per
  // workgroup: a group's shared partitions are read once for all its rows and stream; a row's own
  // token range streams unless a neighbouring row maps its first block too.
  auto run_tiles = [&](auto stream_tag) __attribute__((always_inline)) {
    if (n_mine > 0) {
      // The table entries of the tile after next are asked for before the wait for this tile's data:
      // scalar loads share a counter with the LDS reads, and an outstanding one would hold up the
      // first product (fp8, two heads per wave: 108 -> 100.5 us at batch 64 x 4096 tokens).
      TileT t;
      int ids[4], ids_next[4];
      load_ids(wave, ids);
      issue_as(stream_tag, t, wave, ids);
      if (n_mine > 1) load_ids(wave + W, ids);
      for (int i = 0; i < n_mine; ++i) {
        const int tile = wave + i * W;
        const bool masked = has_tail && tile == ntiles - 1;
        if (i + 2 < n_mine) load_ids(tile + 2 * W, ids_next);
        write_tile(t, tile, masked);
        if (i + 1 < n_mine) issue_as(stream_tag, t, tile + W, ids);
        compute(tile, masked);
#pragma unroll
        for (int x = 0; x < 4; ++x) ids[x] = ids_next[x];
      }
    }
  };
  if (members > 1 || decode_range_is_private(bt_row, p.bt_stride, b, p.batch, min(begin >> p.bs_log2, last_blk)))
    run_tiles(std::true_type{});
  else
    run_tiles(std::false_type{});

  // ---- merge the waves: common reference, then plain sums ---------------------------------------------
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh)
    if (kg == 0) sm[hh * NHC + col][wave] = first ? NEG_INF : m_ref[hh];   // a wave without tiles contributes nothing
  __syncthreads();                                // also: every wave is done with its tiles
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    const float my_ref = first ? NEG_INF : m_ref[hh];
    float mx = sm[hh * NHC + col][0];
#pragma unroll
    for (int i = 1; i < W; ++i) mx = fmaxf(mx, sm[hh * NHC + col][i]);
    const float w = __builtin_amdgcn_exp2f(my_ref - mx);   // exp2(-inf) = 0
    float lw = l_run[hh] * w;
    lw += __shfl_xor(lw, 16);
    lw += __shfl_xor(lw, 32);
    if (kg == 0) sl[hh * NHC + col][wave] = lw;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      *(float4*)&red[wave][(hh * NHC + col) * D + 16 * mt + 4 * kg] =
          make_float4(o[hh][mt][0] * w, o[hh][mt][1] * w, o[hh][mt][2] * w, o[hh][mt][3] * w);
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < HPW * nh * D; idx += W * 64) {
    const int hh = idx / (nh * D);          // KV head of the workgroup
    const int rem = idx - hh * nh * D;
    const int hc = rem / D;                 // head column
    const int d = rem - hc * D;
    const int row_l = hh * NHC + hc;
    float num = 0.0f, den = 0.0f;
#pragma unroll
    for (int i = 0; i < W; ++i) {
      num += red[i][row_l * D + d];
      den += sl[row_l][i];
    }
    const float res = num / den;
    const int head = col_head(hh, hc);
    const int brow = col_row(hc);
    if (p.direct_out) {
      store_from_f32(p.out, brow * p.out_stride + (int64_t)head * D + d, p.q_dtype, res);
    } else {
      const int64_t row = ((int64_t)brow * p.num_q_heads + head) * p.max_partitions + part;
      p.ws_out[row * D + d] = res;
      if (d == 0) {
        float mo = sm[row_l][0];
#pragma unroll
        for (int i = 1; i < W; ++i) mo = fmaxf(mo, sm[row_l][i]);
        p.ws_max[row] = mo * 0.6931471805599453f;  // back to natural-log units
        p.ws_sum[row] = den;
      }
    }
  }
}

template <int KV, int D, int W, int HPW>
static int launch_decode_mfma_one(const DecodeParams& p, dim3 grid, hipStream_t st) {
  constexpr int smem = decode_mfma_lds_bytes(W, HPW, D);
  static_assert(smem <= 160 * 1024, "the tiles of a workgroup must fit the CU's LDS");
  auto kern = paged_decode_mfma_kernel<KV, D, W, HPW>;
  if constexpr (smem > 48 * 1024) {
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

template <int KV, int D>
static int launch_decode_mfma_dim(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st) {
  if (s.hpw == 1) {
    if (s.waves == 8) return launch_decode_mfma_one<KV, D, 8, 1>(p, grid, st);
    if (s.waves == 4) return launch_decode_mfma_one<KV, D, 4, 1>(p, grid, st);
    if (s.waves == 2) return launch_decode_mfma_one<KV, D, 2, 1>(p, grid, st);
  } else if (s.hpw == 2) {
    if (s.waves == 4) return launch_decode_mfma_one<KV, D, 4, 2>(p, grid, st);
    if (s.waves == 2) return launch_decode_mfma_one<KV, D, 2, 2>(p, grid, st);
  }
  return fail(PA_ERR_UNSUPPORTED, "pa_decode: the matrix path takes 2, 4 or 8 waves per workgroup with one KV head per wave, 2 or 4 with two");
}

template <int KV>
static int launch_decode_mfma(const DecodeParams& p, dim3 grid, const DecodeShape& s, hipStream_t st) {
  if (s.head_dim == 128) return launch_decode_mfma_dim<KV, 128>(p, grid, s, st);
  if (s.head_dim == 64) return launch_decode_mfma_dim<KV, 64>(p, grid, s, st);
  return fail(PA_ERR_UNSUPPORTED, "pa_decode: head_dim must be 64 or 128");
}

}  // namespace pa
