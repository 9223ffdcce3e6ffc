// Chunked-prefill paged attention for gfx950 on the MFMA matrix cores.
//
// Reference semantics: PagedAttention._prefill_attention (src/inference/attention.py:240-261):
// flash_attn_varlen_func(q, k_src, v_src, cu_seqlens_q, cu_seqlens_k, causal=True,
// block_table=...) where K/V come from the paged cache when a prefix is cached, else from the
// new tokens themselves; the causal mask is bottom-right aligned (row i of a chunk of Lq rows
// sees keys 0 .. Lk-Lq+i).  Without a prefix this is _sdpa_prefill_fallback (:281-315).
//
// Here QK^T and PV are real dense tiles, so they run on v_mfma_f32_32x32x16_f16 with fp32
// accumulation:
//
//  * One workgroup of W = 4 or 8 waves owns 32 W query rows that share one KV head: 16 W tokens x
//    the two query heads of a GQA pair (or 32 W tokens x 1 head).  Each wave owns 32 rows and
//    keeps their Q as MFMA B operands in registers for the whole kernel.  W = 8 puts twice the
//    rows behind every K/V tile, which halves the bytes a CU pulls through its L1; large launches
//    use it.
//  * The KV sequence is walked in tiles of 64 keys.  A tile of K and of V (64 x head_dim) is
//    fetched through the block table with 16-byte coalesced loads, converted to fp16 if the cache
//    is bf16 / fp8 (fp8: value / per-token scale), and staged in LDS in its natural [key][dim]
//    layout; LDS is double buffered so the loads of tile t+1 are in flight while tile t is
//    multiplied.  All waves read the same tile: every K/V byte is fetched once per 32 W rows.
//  * S^T = K . Q^T (keys x queries) rather than S: in the MFMA result layout a lane then holds 16
//    keys of ONE query, so the online-softmax row max / row sum are in-lane reductions plus a
//    single exchange with lane^32, and the fp16 probabilities are already laid out as the B
//    operand of the next product.
//  * O^T = V^T . P^T: the A operand needs 8 keys of one head_dim column per lane, i.e. V
//    transposed.  V stays untransposed in LDS and is read with ds_read_b64_tr_b16, the LDS
//    transpose load of gfx950 (16 lanes read a 4-key x 16-dim patch and each gets the 4 keys of
//    its own column).  The two 4-key groups a lane fetches are the keys the S^T layout gives that
//    lane half, so no shuffle sits between the two products.
//  * The softmax costs a lane an exp2, half a conversion, half a dot-2 add and a third of a max per
//    score: Q is multiplied by scale * log2(e) once, on its way into fp16; the score products
//    start from a block of registers holding minus the row's reference point, so the matrix pipe
//    delivers exp2 arguments; probabilities are converted to fp16 in pairs and the row sum adds
//    those pairs (v_dot2c_f32_f16 with ones), i.e. exactly what the second product multiplies;
//    the two lane halves of a query column compare maxima with one v_permlane32_swap.
//  * The mask is applied only on tiles that cross the diagonal or the end of the sequence.
#include "pa_common.hpp"
#include "pa_host.hpp"

#include <math.h>
#include <stdio.h>

#include <atomic>
#include <type_traits>
#include <utility>

namespace pa {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2v_t __attribute__((ext_vector_type(2)));
typedef unsigned uint2v_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));

struct PrefillParams {
  const void* q;
  int64_t q_stride;
  const uint8_t* k;  // paged cache [num_blocks, block_size, kv_heads, D] or dense [tokens, kv_heads, D]
  const uint8_t* v;
  const float* k_scale;
  const float* v_scale;
  const int32_t* block_tables;  // nullptr = dense K/V indexed by cu_seqlens_k
  int64_t bt_stride;
  int64_t kv_token_stride;  // dense mode: elements between consecutive tokens
  const int32_t* cu_q;
  const int32_t* cu_k;
  void* out;
  int64_t out_stride;
  int q_dtype;
  int num_q_heads;
  int num_kv_heads;
  int bs_log2;
  int num_blocks;
  float scale_log2e;
};

enum : int { SRC_F16 = 0, SRC_BF16 = 1, SRC_FP8 = 2, SRC_F32 = 3 };

constexpr int kBN = 64;  // keys per tile
constexpr int kMaxDevices = 64;

// LDS reads of the tile loop, issued as opaque asm.  ds_read_b64_tr_b16 is the LDS transpose load
// of gfx950: within each block of 16 lanes, lane i receives element (i % 4) of the 8 bytes
// addressed by lanes 4j + i/4, j = 0..3 (checked on hardware).  Left to the compiler, every read
// is followed by a wait and the product that uses it (ds_read -> s_waitcnt -> mfma, one k-step at a
// time), and its wait-count pass, which cannot tell that a transpose read does not touch the
// buffer that global_load_lds is filling, drains every outstanding global load in front of it.
// The result of an untracked read is not known to that pass: the caller waits with lds_wait<N>
// before use.  LDS operations complete in order, so the extra outstanding reads only make the
// compiler's own lgkmcnt waits more conservative.
template <int OFF>
__device__ __forceinline__ half4_t tr_read_untracked(uint32_t lds_byte_addr) {
  half4_t r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(lds_byte_addr), "n"(OFF));
  return r;
}
template <int OFF>
__device__ __forceinline__ half8_t b128_read_untracked(uint32_t lds_byte_addr) {
  half8_t r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(lds_byte_addr), "n"(OFF));
  return r;
}
// Waits until at most N LDS operations are outstanding; the operands are tied so that no consumer
// of them can be scheduled above the wait.
template <int N>
__device__ __forceinline__ void lds_wait(half4_t& a, half4_t& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_wait(half8_t& a, half8_t& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// One stage of a K or V tile in LDS: [key][head_dim] fp16 rows with no padding; the 16-byte
// chunk c of row r lives at chunk position c ^ swz(r).  swz swaps the two low bit pairs of the
// row number, so that (a) 16 consecutive rows get 16 different values: the 16 lanes that read
// the same chunk index of 16 rows (MFMA A-operand reads of K) hit distinct banks, and (b) 4
// consecutive rows differ in bits 2..3: the 4-row x 64-byte patch that 32 lanes fetch in one
// pass of a transpose read of V spreads over 16 distinct chunk positions.
template <int CPR>
__device__ __forceinline__ constexpr int swz(int row) {
  return (((row & 3) << 2) | ((row >> 2) & 3)) & (CPR - 1);
}

template <int D>
struct PrefillLds {
  _Float16 k[2][kBN * D];
  _Float16 v[2][kBN * D];
};

// 8 consecutive source elements as loaded.  The staging registers hold them in this form while the
// tile before is being multiplied, so that nothing waits for the load until the tile is committed.
// (fp32 sources are the exception: 8 registers per chunk would not fit beside the accumulators, so
// they are converted as they arrive and staged as fp16.)
template <int SRC> struct RawChunk { uint4 a; };
template <> struct RawChunk<SRC_FP8> { uint2 a; };

template <int SRC>
__device__ __forceinline__ RawChunk<SRC> load8_raw(const uint8_t* p) {
  RawChunk<SRC> r;
  if constexpr (SRC == SRC_FP8) {
    r.a = *(const uint2*)p;
  } else if constexpr (SRC == SRC_F32) {
    const float4 a = *(const float4*)p;
    const float4 b = *(const float4*)(p + 16);
    const half8_t h = {(_Float16)a.x, (_Float16)a.y, (_Float16)a.z, (_Float16)a.w,
                       (_Float16)b.x, (_Float16)b.y, (_Float16)b.z, (_Float16)b.w};
    __builtin_memcpy(&r.a, &h, 16);
  } else {
    r.a = *(const uint4*)p;
  }
  return r;
}

// 8 loaded source elements -> 8 fp16 (fp8: times inv_scale = 1 / the token's scale)
template <int SRC>
__device__ __forceinline__ half8_t raw_to_f16(const RawChunk<SRC>& w, float inv_scale) {
  half8_t r;
  if constexpr (SRC == SRC_F16 || SRC == SRC_F32) {
    __builtin_memcpy(&r, &w.a, 16);
  } else if constexpr (SRC == SRC_BF16) {
    const uint32_t ww[4] = {w.a.x, w.a.y, w.a.z, w.a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      r[2 * i] = (_Float16)__uint_as_float(ww[i] << 16);
      r[2 * i + 1] = (_Float16)__uint_as_float(ww[i] & 0xffff0000u);
    }
  } else if constexpr (SRC == SRC_FP8) {
    // byte / scale = byte * m * 2^e with m in [1, 2): v_cvt_scalef32_pk_f16_fp8 applies the power of
    // two exactly while it converts a pair, and the mantissa is one packed fp16 multiply per pair
    // (8 vector instructions per 8 elements instead of 20 through fp32)
    const uint32_t ww[2] = {w.a.x, w.a.y};
    const uint32_t bits = __float_as_uint(inv_scale);
    const float pow2 = __uint_as_float(bits & 0xff800000u);
    const _Float16 m = (_Float16)__uint_as_float((bits & 0x007fffffu) | 0x3f800000u);
    const half2v_t mm = {m, m};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const half2v_t lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(ww[i], pow2, false) * mm;
      const half2v_t hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(ww[i], pow2, true) * mm;
      r[4 * i] = lo[0];
      r[4 * i + 1] = lo[1];
      r[4 * i + 2] = hi[0];
      r[4 * i + 3] = hi[1];
    }
  }
  return r;
}

template <int SRC>
constexpr int src_bytes() { return SRC == SRC_FP8 ? 1 : (SRC == SRC_F32 ? 4 : 2); }

// DIRECT: fp16 sources go global -> LDS with global_load_lds_dwordx4 (no staging registers); other
// source types are converted in registers on the way.  W = waves per workgroup: 4 (two workgroups
// per CU) or 8 (one, with twice the query rows behind every K/V tile).
template <int D, int HPWG, int SRC, int W>
__global__ __launch_bounds__(64 * W, (W == 4 ? 2 : 1)) void paged_prefill_kernel(const PrefillParams p) {
  constexpr int NT = 64 * W;              // threads per workgroup
  using L = PrefillLds<D>;
  constexpr bool DIRECT = SRC == SRC_F16;
  constexpr int KSTEPS = D / 16;          // MFMA k-steps over head_dim
  constexpr int MT = D / 32;              // 32-row tiles of O^T
  constexpr int BM = 32 * W / HPWG;       // query tokens per workgroup
  constexpr int CPR = D / 8;              // 8-element chunks per row
  constexpr int NCH = kBN * CPR / NT;     // chunks per thread per tile (K and V each)
  constexpr int ES = src_bytes<SRC>();
  constexpr float NEG_INF = -INFINITY;

  extern __shared__ __align__(16) uint8_t smem_raw[];
  L& lds = *reinterpret_cast<L*>(smem_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31;   // query column of this lane
  const int h = lane >> 5;   // lane half: which 8 of the 16 k-slots
  const int seq = blockIdx.z;
  const int q0 = p.cu_q[seq];
  const int lq = p.cu_q[seq + 1] - q0;
  const int k0 = p.cu_k[seq];
  const int lk = p.cu_k[seq + 1] - k0;
  // blockIdx.x (fastest, dealt round-robin to the 8 XCDs) is the head group: all query tiles of
  // one KV head then run on the same XCD and share its L2, so a K/V tile is fetched from HBM
  // once instead of once per query tile.
  // Query tiles are handed out last first: under the causal mask the last tile of a sequence has
  // the most keys, and when a launch has more workgroups than the GPU holds at once the long ones
  // should start first and the short ones fill the end.
  const int tok0 = (int)(gridDim.y - 1 - blockIdx.y) * BM;
  if (tok0 >= lq) return;
  const int shift = lk - lq;  // row i sees keys <= i + shift

  const int hslot = (HPWG == 2) ? wave / (W / 2) : 0;
  const int tsub = (HPWG == 2) ? wave % (W / 2) : wave;
  const int qhead = blockIdx.x * HPWG + hslot;
  const int kvh = (blockIdx.x * HPWG) / (p.num_q_heads / p.num_kv_heads);
  const int tokw0 = tok0 + tsub * 32;            // first token of this wave
  const int tok = tokw0 + n;                     // this lane's token
  const bool row_ok = tok < lq;
  const int qlim = tok + shift;                  // last visible key of this lane's row

  // ---- Q as B operands: [d-step][8 halfs], loaded once ------------------------------------------
  half8_t qreg[KSTEPS];
  {
    const int tq = min(tok, lq - 1);
    const int64_t base = (int64_t)(q0 + tq) * p.q_stride + (int64_t)qhead * D + 8 * h;
    // the dtype switch sits outside the loop: inside, it would put a branch and a wait between
    // loads that are meant to be in flight together
    auto load_q = [&](auto dt_tag) __attribute__((always_inline)) {
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        float x[8];
        load8_as_f32(p.q, base + ks * 16, decltype(dt_tag)::value, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) qreg[ks][e] = (_Float16)(x[e] * p.scale_log2e);
      }
    };
    if (p.q_dtype == PA_DTYPE_F16) load_q(std::integral_constant<int, PA_DTYPE_F16>{});
    else if (p.q_dtype == PA_DTYPE_BF16) load_q(std::integral_constant<int, PA_DTYPE_BF16>{});
    else load_q(std::integral_constant<int, PA_DTYPE_F32>{});
  }

  float16_t o[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[mt][i] = 0.0f;
  float l_run = 0.0f;     // running sum of this lane half's probabilities
  // Q carries scale * log2(e), and the first product of every score tile starts from the block
  // neg_ref (-m_ref in all 16 registers) instead of zero: the matrix pipe hands back
  // s * scale * log2(e) - m_ref, ready for exp2, and the softmax needs no multiply-add per score.
  float m_ref = 0.0f;     // reference point of the exponentials (same in both lane halves)
  float16_t neg_ref;
#pragma unroll
  for (int i = 0; i < 16; ++i) neg_ref[i] = 0.0f;

  // keys the workgroup needs: up to the last valid row's limit
  const int last_tok = min(tok0 + BM, lq) - 1;
  const int kend = min(lk, last_tok + shift + 1);
  const int ntiles = (kend + kBN - 1) / kBN;
  // this wave's last visible key (wave-uniform)
  const int wave_last = min(tokw0 + 31, lq - 1) + shift;
  const bool wave_has_rows = tokw0 < lq;

  const int bs_mask = (1 << p.bs_log2) - 1;
  const int64_t token_elems = p.block_tables ? (int64_t)p.num_kv_heads * D : p.kv_token_stride;
  const uint32_t row_bytes = (uint32_t)(token_elems * ES);      // bytes between consecutive tokens (the host checks the range)
  const int32_t* bt_row = p.block_tables ? p.block_tables + seq * p.bt_stride : nullptr;
  const int bt_last = max((int)p.bt_stride - 1, 0);

  // ---- staging: global -> (registers ->) LDS ---------------------------------------------------------
  // chunk = 16 bytes of fp16 = 8 head-dim elements; thread `tid` moves chunks tid, tid+NT, ...
  // i.e. one instruction of a wave covers 64 / CPR whole rows, contiguous in LDS.
  auto row_slot = [&](int key) __attribute__((always_inline)) -> int64_t {   // physical row of a key (clamped: never faults)
    const int kk = min(key, lk - 1);
    if (bt_row) {
      const int blk = min(kk >> p.bs_log2, bt_last);
      const int phys = min(max(bt_row[blk], 0), p.num_blocks - 1);
      return ((int64_t)phys << p.bs_log2) + (kk & bs_mask);
    }
    return (int64_t)k0 + kk;
  };
  RawChunk<SRC> stage_k[DIRECT ? 1 : NCH], stage_v[DIRECT ? 1 : NCH];
  float stage_ks[SRC == SRC_FP8 ? NCH : 1], stage_vs[SRC == SRC_FP8 ? NCH : 1];   // the tokens' scales, as loaded
  // Fast path for tiles that lie wholly inside the sequence: the 64/CPR rows one wave moves per
  // instruction belong to one block (block_size >= 16) or are consecutive dense rows, so the
  // row base is wave-uniform (scalar table load, scalar 64-bit base) and the per-lane part of
  // the address never changes between tiles.
  const bool uniform_rows = bt_row == nullptr || p.bs_log2 >= 4;
  uint32_t lane_part[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int chunk = tid + NT * c;
    const int row = chunk / CPR;
    const int col = (chunk % CPR) ^ swz<CPR>(row);
    lane_part[c] = (uint32_t)(((lane / CPR) * token_elems + (int64_t)kvh * D + col * 8) * ES);
  }
  auto move_chunk = [&](int c, int buf, const uint8_t* kp, const uint8_t* vp, int64_t slot) __attribute__((always_inline)) {
    if constexpr (DIRECT) {
      const int wbase = (NT * c + wave * 64) * 8;     // LDS destination = wave base + lane * 16 bytes
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)kp,
                                       (__attribute__((address_space(3))) void*)&lds.k[buf][wbase], 16, 0, 0);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)vp,
                                       (__attribute__((address_space(3))) void*)&lds.v[buf][wbase], 16, 0, 0);
    } else {
      if constexpr (SRC == SRC_FP8) {
        stage_ks[c] = p.k_scale[slot];
        stage_vs[c] = p.v_scale[slot];
      }
      stage_k[c] = load8_raw<SRC>(kp);
      stage_v[c] = load8_raw<SRC>(vp);
    }
  };
  // Block-table entries of a tile, fetched one tile ahead of the loads that need them so that no
  // load ever waits on another: lane l holds the entry of chunk group l % NCH of this wave.
  auto load_ids = [&](int t) __attribute__((always_inline)) -> int {
    if (!bt_row) return 0;
    const int row0 = (NT * (lane % NCH) + 64 * wave) / CPR;
    return bt_row[min((t * kBN + row0) >> p.bs_log2, bt_last)];
  };
  // wave-uniform 64-bit pointer in scalar registers: with the lane's constant 32-bit offset added
  // the load takes the "scalar base + vector offset" form
  auto uniform_ptr = [](const uint8_t* q) __attribute__((always_inline)) {
    const uint64_t a = (uint64_t)(uintptr_t)q;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
    return (const uint8_t*)(uintptr_t)(((uint64_t)hi << 32) | lo);
  };
  auto fetch = [&](int t, int buf, int ids) __attribute__((always_inline)) {
    if (uniform_rows && (t + 1) * kBN <= lk) {
      // straight-line code per addressing mode: the waves of a workgroup leave the barrier together
      // and fetch the same instructions, and every taken branch costs each of them a refill
      if (bt_row) {
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
          const int key0 = t * kBN + (NT * c) / CPR + wave * (64 / CPR);   // first row of this wave's instruction
          const int phys = min(max(__builtin_amdgcn_readlane(ids, c), 0), p.num_blocks - 1);
          const int64_t slot0 = ((int64_t)phys << p.bs_log2) + (key0 & bs_mask);
          const uint64_t base = (uint64_t)(uint32_t)slot0 * row_bytes;     // both below 2^32: one 32 x 32 -> 64 multiply
          move_chunk(c, buf, uniform_ptr(p.k + base) + lane_part[c], uniform_ptr(p.v + base) + lane_part[c], slot0 + lane / CPR);
        }
      } else {
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
          const int key0 = t * kBN + (NT * c) / CPR + wave * (64 / CPR);
          const int64_t slot0 = (int64_t)k0 + key0;
          const uint64_t base = (uint64_t)(uint32_t)slot0 * row_bytes;
          move_chunk(c, buf, uniform_ptr(p.k + base) + lane_part[c], uniform_ptr(p.v + base) + lane_part[c], slot0 + lane / CPR);
        }
      }
      return;
    }
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int chunk = tid + NT * c;
      const int row = chunk / CPR;
      const int col = (chunk % CPR) ^ swz<CPR>(row);   // head-dim chunk that belongs at this LDS position
      const int64_t slot = row_slot(t * kBN + row);    // rows past the sequence end re-read its last row (masked later)
      const int64_t eoff = (slot * token_elems + (int64_t)kvh * D + col * 8) * ES;
      move_chunk(c, buf, p.k + eoff, p.v + eoff, slot);
    }
  };
  auto commit = [&](int buf) __attribute__((always_inline)) {
    if constexpr (!DIRECT) {
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int chunk = tid + NT * c;
        float iks = 1.0f, ivs = 1.0f;
        if constexpr (SRC == SRC_FP8) {
          iks = __builtin_amdgcn_rcpf(stage_ks[c]);
          ivs = __builtin_amdgcn_rcpf(stage_vs[c]);
        }
        *(half8_t*)&lds.k[buf][chunk * 8] = raw_to_f16<SRC>(stage_k[c], iks);
        *(half8_t*)&lds.v[buf][chunk * 8] = raw_to_f16<SRC>(stage_v[c], ivs);
      }
    }
  };

  // ---- loop-invariant LDS read offsets (in halfs, before the buffer / tile-row offsets) ------------
  // S^T A operand: key row n of a 32-key tile, head-dim chunk 2*ks + h
  int k_off[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) k_off[ks] = n * D + (((2 * ks + h) ^ swz<CPR>(n)) << 3);
  // O^T A operand through the transpose read: lanes form 4 blocks of 16 = (dim half of the
  // 32-row tile, lane half); inside a block lane i supplies the address of key (i/4), dims
  // 4*(i%4).. and receives the 4 keys of dim i.  lo/hi = the two 4-key groups of a 16-key step
  // that the S^T result layout gives this lane half: keys 4h.. and 8+4h..
  const int tr_i = lane & 15;
  const int tr_dblk = (lane >> 4) & 1;
  int v_off[MT][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int row = 8 * r + 4 * h + (tr_i >> 2);                     // row & 15 of the key
      const int chunk = 4 * mt + 2 * tr_dblk + ((tr_i & 3) >> 1);      // head-dim chunk
      v_off[mt][r] = row * D + ((chunk ^ swz<CPR>(row)) << 3) + 4 * (tr_i & 1);
    }

  const uint32_t k_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)&lds.k[0][0];
  uint32_t k_addr[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) k_addr[ks] = k_base + 2u * (uint32_t)k_off[ks];
  const uint32_t v_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)&lds.v[0][0];
  uint32_t v_addr[MT][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int r = 0; r < 2; ++r) v_addr[mt][r] = v_base + 2u * (uint32_t)v_off[mt][r];

  // `buf` is a compile-time constant (the tile loop is unrolled by two) so that every LDS read
  // below is "loop-invariant register + immediate offset".
  auto compute = [&](int t, auto buf_tag) __attribute__((always_inline)) {
    constexpr int buf = decltype(buf_tag)::value;
    const int kt0 = t * kBN;
    // ---- S^T = K . Q^T : two 32-key tiles -------------------------------------------------------
    float16_t s[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[kt][i] = neg_ref[i];
    // All K fragments of the first 32-key half are requested at once and those of the second
    // half as the first are consumed, so a product never waits for a read issued just before it.
    constexpr int OFF0 = buf * kBN * D * 2, OFF1 = OFF0 + 32 * D * 2;
    half8_t ka[KSTEPS], kb[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) ka[ks] = b128_read_untracked<OFF0>(k_addr[ks]);
    static_for<KSTEPS / 2>([&](auto j_tag) __attribute__((always_inline)) {
      constexpr int ks = 2 * decltype(j_tag)::value;
      lds_wait<KSTEPS - 2>(ka[ks], ka[ks + 1]);   // outstanding: the rest of ka and what is issued of kb
      s[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[ks], qreg[ks], s[0], 0, 0, 0);
      s[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[ks + 1], qreg[ks + 1], s[0], 0, 0, 0);
      kb[ks] = b128_read_untracked<OFF1>(k_addr[ks]);
      kb[ks + 1] = b128_read_untracked<OFF1>(k_addr[ks + 1]);
    });
    static_for<KSTEPS / 2>([&](auto j_tag) __attribute__((always_inline)) {
      constexpr int ks = 2 * decltype(j_tag)::value;
      lds_wait<KSTEPS - 2 - ks>(kb[ks], kb[ks + 1]);
      s[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kb[ks], qreg[ks], s[1], 0, 0, 0);
      s[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kb[ks + 1], qreg[ks + 1], s[1], 0, 0, 0);
    });
    // ---- mask: only tiles that reach past the diagonal of this wave or the sequence end ---------
    const int wave_first_lim = tokw0 + shift;  // smallest row limit in the wave
    if (kt0 + kBN - 1 > wave_first_lim || kt0 + kBN > lk) {
      const int lim = min(qlim, lk - 1);
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = kt0 + kt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
          s[kt][i] = key <= lim ? s[kt][i] : NEG_INF;
        }
    }
    half8_t pb[4];
    {
      // ---- online softmax over this lane's query column; the scores arrive in the exponent domain,
      // relative to m_ref ---------------------------------------------------------------------------
      float mloc = s[0][0];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, s[kt][i]);
      {
        // the other 16 keys of this query column sit 32 lanes away
        const uint2v_t sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mloc), __float_as_uint(mloc), false, false);
        mloc = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
      }
      // Lazy rescale: the first tile sets the reference to its maximum; later it only follows the
      // true maximum when that has outgrown it by more than 2^8, so probabilities stay <= 256
      // (exact enough in fp16 and fp32) and the rescale of the 64 accumulator registers, of this
      // tile's scores and of the reference block almost never runs.  The final division by the
      // row sum removes whatever reference point was used.  A row with no visible key yet (all
      // scores -inf) keeps reference 0 and adds nothing.
      const bool grow = (t == 0) ? (mloc > NEG_INF) : (mloc > 8.0f);
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(grow) != 0, 0)) {
        const float delta = grow ? mloc : 0.0f;
        const float alpha = (t == 0) ? 1.0f : __builtin_amdgcn_exp2f(-delta);   // accumulators are zero on the first tile
        l_run *= alpha;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[mt][i] *= alpha;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) s[kt][i] -= delta;
        m_ref += delta;
#pragma unroll
        for (int i = 0; i < 16; ++i) neg_ref[i] = -m_ref;
      }
      float psum = 0.0f;
      const half2v_t one2 = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const half2v_t h = {(_Float16)__builtin_amdgcn_exp2f(s[kt][i]), (_Float16)__builtin_amdgcn_exp2f(s[kt][i + 1])};
          psum = __builtin_amdgcn_fdot2(h, one2, psum, false);   // the row sum adds what the second product multiplies
          pb[kt * 2 + (i >> 3)][i & 7] = h[0];
          pb[kt * 2 + (i >> 3)][(i & 7) + 1] = h[1];
        }
      l_run += psum;
    }
    // ---- O^T += V^T . P^T : four 16-key steps x MT row tiles ----------------------------------------
    // untracked reads, one 16-key step ahead of the products that use them
    half4_t lo[2][MT], hi[2][MT];
    auto issue = [&](auto k2_tag) __attribute__((always_inline)) {
      constexpr int k2 = decltype(k2_tag)::value;
      constexpr int OFF = (buf * kBN * D + k2 * 16 * D) * 2;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        lo[k2 & 1][mt] = tr_read_untracked<OFF>(v_addr[mt][0]);
        hi[k2 & 1][mt] = tr_read_untracked<OFF>(v_addr[mt][1]);
      }
    };
    auto multiply = [&](auto k2_tag) __attribute__((always_inline)) {
      constexpr int k2 = decltype(k2_tag)::value;
      // reads return in order: this step's have all landed once no more than the next step's
      // 2 MT are outstanding.  volatile asm statements keep their order, so tying the other
      // registers to empty statements after the wait holds their consumers below it too.
      if constexpr (k2 < 3) lds_wait<2 * MT>(lo[k2 & 1][0], hi[k2 & 1][0]);
      else lds_wait<0>(lo[k2 & 1][0], hi[k2 & 1][0]);
#pragma unroll
      for (int mt = 1; mt < MT; ++mt) asm volatile("" : "+v"(lo[k2 & 1][mt]), "+v"(hi[k2 & 1][mt]));
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const half4_t l4 = lo[k2 & 1][mt], h4 = hi[k2 & 1][mt];
        half8_t a;
        a[0] = l4[0]; a[1] = l4[1]; a[2] = l4[2]; a[3] = l4[3];
        a[4] = h4[0]; a[5] = h4[1]; a[6] = h4[2]; a[7] = h4[3];
        o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[k2], o[mt], 0, 0, 0);
      }
    };
    issue(std::integral_constant<int, 0>{});
    issue(std::integral_constant<int, 1>{});
    multiply(std::integral_constant<int, 0>{});
    issue(std::integral_constant<int, 2>{});
    multiply(std::integral_constant<int, 1>{});
    issue(std::integral_constant<int, 3>{});
    multiply(std::integral_constant<int, 2>{});
    multiply(std::integral_constant<int, 3>{});
  };

  // ---- tile loop: LDS double buffer, one barrier per tile -------------------------------------------
  int ids = 0;
  if (ntiles > 0) {
    ids = load_ids(0);
    fetch(0, 0, ids);
    commit(0);
    if (ntiles > 1) ids = load_ids(1);
  }
  __syncthreads();
  auto step = [&](int t, auto buf_tag) __attribute__((always_inline)) {
    constexpr int buf = decltype(buf_tag)::value;
    const bool more = t + 1 < ntiles;
    if (more) {
      fetch(t + 1, buf ^ 1, ids);      // direct loads land in the other buffer while this one is used
      if (t + 2 < ntiles) ids = load_ids(t + 2);
    }
    if (wave_has_rows && t * kBN <= wave_last) compute(t, buf_tag);
    if (more) commit(buf ^ 1);
    __syncthreads();                   // also waits for this wave's outstanding loads into LDS
  };
  for (int t = 0; t < ntiles; t += 2) {
    step(t, std::integral_constant<int, 0>{});
    if (t + 1 < ntiles) step(t + 1, std::integral_constant<int, 1>{});
  }

  // ---- normalise and store ---------------------------------------------------------------------------
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  if (!row_ok) return;
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  const int64_t obase = (int64_t)(q0 + tok) * p.out_stride + (int64_t)qhead * D;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const int d = 32 * mt + 8 * g4 + 4 * h;
      const float x0 = o[mt][4 * g4] * inv, x1 = o[mt][4 * g4 + 1] * inv;
      const float x2 = o[mt][4 * g4 + 2] * inv, x3 = o[mt][4 * g4 + 3] * inv;
      if (p.q_dtype == PA_DTYPE_F32) {
        *(float4*)((float*)p.out + obase + d) = make_float4(x0, x1, x2, x3);
      } else if (p.q_dtype == PA_DTYPE_F16) {
        uint2 w;
        w.x = (uint32_t)f32_to_f16_bits(x0) | ((uint32_t)f32_to_f16_bits(x1) << 16);
        w.y = (uint32_t)f32_to_f16_bits(x2) | ((uint32_t)f32_to_f16_bits(x3) << 16);
        *(uint2*)((uint16_t*)p.out + obase + d) = w;
      } else {
        uint2 w;
        w.x = (uint32_t)f32_to_bf16_bits(x0) | ((uint32_t)f32_to_bf16_bits(x1) << 16);
        w.y = (uint32_t)f32_to_bf16_bits(x2) | ((uint32_t)f32_to_bf16_bits(x3) << 16);
        *(uint2*)((uint16_t*)p.out + obase + d) = w;
      }
    }
}

template <int D, int HPWG, int SRC, int W>
static int launch_prefill(const PrefillParams& p, dim3 grid, hipStream_t st) {
  auto kern = paged_prefill_kernel<D, HPWG, SRC, W>;
  const size_t smem = sizeof(PrefillLds<D>);
  // the attribute belongs to the kernel on one device: once per instantiation and device
  static std::atomic<bool> attr_set[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(PA_ERR_LAUNCH, "pa_prefill: cannot tell the current device");
  if (!attr_set[dev].load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
      return fail(PA_ERR_LAUNCH, "pa_prefill: cannot raise the dynamic LDS limit");
    attr_set[dev].store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, grid, dim3(64 * W), smem, st, p);
  return PA_OK;
}

template <int D, int HPWG, int W>
static int launch_prefill_src(const PrefillParams& p, dim3 grid, int src, hipStream_t st) {
  switch (src) {
    case SRC_F16: return launch_prefill<D, HPWG, SRC_F16, W>(p, grid, st);
    case SRC_BF16: return launch_prefill<D, HPWG, SRC_BF16, W>(p, grid, st);
    case SRC_FP8: return launch_prefill<D, HPWG, SRC_FP8, W>(p, grid, st);
    default: return launch_prefill<D, HPWG, SRC_F32, W>(p, grid, st);
  }
}

template <int D, int W>
static int launch_prefill_hpwg(const PrefillParams& p, dim3 grid, int hpwg, int src, hipStream_t st) {
  return hpwg == 2 ? launch_prefill_src<D, 2, W>(p, grid, src, st) : launch_prefill_src<D, 1, W>(p, grid, src, st);
}

}  // namespace pa

using namespace pa;

extern "C" int pa_prefill(const void* q, int q_dtype, int64_t q_token_stride, const void* k_cache,
                          const void* v_cache, const float* k_scale, const float* v_scale,
                          int kv_dtype, const int32_t* block_tables, int64_t bt_stride,
                          const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, void* out,
                          int64_t out_token_stride, int64_t num_seqs, int64_t max_seqlen_q,
                          int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                          int64_t block_size, int64_t num_blocks, float scale,
                          int waves_per_workgroup, void* stream) {
  if (waves_per_workgroup != 0 && waves_per_workgroup != 4 && waves_per_workgroup != 8)
    return fail(PA_ERR_BAD_ARG, "pa_prefill: waves_per_workgroup must be 0 (automatic), 4 or 8");
  if (num_seqs < 0 || max_seqlen_q < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0)
    return fail(PA_ERR_BAD_ARG, "pa_prefill: negative or zero size");
  if (num_seqs == 0 || max_seqlen_q == 0) return PA_OK;
  if (!q || !k_cache || !v_cache || !cu_seqlens_q || !cu_seqlens_k || !out)
    return fail(PA_ERR_BAD_ARG, "pa_prefill: null pointer");
  if (q_dtype != PA_DTYPE_F16 && q_dtype != PA_DTYPE_BF16 && q_dtype != PA_DTYPE_F32)
    return fail(PA_ERR_UNSUPPORTED, "pa_prefill: q_dtype must be f16, bf16 or f32");
  int src;
  switch (kv_dtype) {
    case PA_DTYPE_F16: src = SRC_F16; break;
    case PA_DTYPE_BF16: src = SRC_BF16; break;
    case PA_DTYPE_FP8_E4M3: src = SRC_FP8; break;
    case PA_DTYPE_F32: src = SRC_F32; break;
    default: return fail(PA_ERR_UNSUPPORTED, "pa_prefill: kv_dtype must be f16, bf16, f32 or fp8-e4m3");
  }
  if (src == SRC_FP8 && (!k_scale || !v_scale))
    return fail(PA_ERR_BAD_ARG, "pa_prefill: fp8 cache needs k_scale and v_scale");
  if (src == SRC_FP8 && !block_tables)
    return fail(PA_ERR_UNSUPPORTED, "pa_prefill: fp8 K/V need the paged cache (block_tables)");
  if (head_dim != 64 && head_dim != 128)
    return fail(PA_ERR_UNSUPPORTED, "pa_prefill: head_dim must be 64 or 128");
  if (!(scale > 0.0f) || scale > 3.0e38f)
    return fail(PA_ERR_BAD_ARG, "pa_prefill: scale must be positive and finite (masked scores are -inf times scale)");
  if (num_q_heads % num_kv_heads != 0)
    return fail(PA_ERR_BAD_ARG, "pa_prefill: num_q_heads must be a multiple of num_kv_heads");
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out))
    return fail(PA_ERR_BAD_ARG, "pa_prefill: buffers must be 16-byte aligned");
  if (q_token_stride < num_q_heads * head_dim || out_token_stride < num_q_heads * head_dim ||
      q_token_stride % 8 != 0 || out_token_stride % 4 != 0)
    return fail(PA_ERR_BAD_ARG, "pa_prefill: bad q/out token stride");
  int bs_log2 = 0;
  int64_t kv_token_stride = 0;
  if (block_tables) {
    if (block_size <= 0 || (block_size & (block_size - 1)) != 0)
      return fail(PA_ERR_UNSUPPORTED, "pa_prefill: block_size must be a power of two");
    while ((int64_t(1) << bs_log2) < block_size) ++bs_log2;
    if (num_blocks <= 0 || bt_stride <= 0) return fail(PA_ERR_BAD_ARG, "pa_prefill: bad pool or table size");
  } else {
    // dense K/V [total_k_tokens, kv_heads, head_dim]: bt_stride carries the token stride in elements
    kv_token_stride = bt_stride > 0 ? bt_stride : num_kv_heads * head_dim;
    if (kv_token_stride < num_kv_heads * head_dim || kv_token_stride % 8 != 0)
      return fail(PA_ERR_BAD_ARG, "pa_prefill: bad dense K/V token stride");
    num_blocks = 1;
  }
  if (num_seqs > 65535 || max_seqlen_q > 65535 * 64)
    return fail(PA_ERR_UNSUPPORTED, "pa_prefill: too many sequences or query tokens for one launch");
  // the kernel multiplies a token's slot by the bytes between tokens as two 32-bit numbers
  if (num_blocks * block_size >= (int64_t(1) << 32) || kv_token_stride >= (int64_t(1) << 30) ||
      num_kv_heads * head_dim >= (int64_t(1) << 30))
    return fail(PA_ERR_UNSUPPORTED, "pa_prefill: pool of 2^32 slots or more, or 2^30 elements or more between tokens");

  const int g = (int)(num_q_heads / num_kv_heads);
  const int hpwg = (g % 2 == 0) ? 2 : 1;
  // 8 waves per workgroup share each K/V tile between twice as many query rows, which halves
  // the bytes every CU pulls through its L1; worth it once such workgroups fill most of the chip.
  int w = waves_per_workgroup;
  if (w == 0) {
    const int64_t bm8 = 256 / hpwg;
    const int64_t wgs8 = (num_q_heads / hpwg) * ((max_seqlen_q + bm8 - 1) / bm8) * num_seqs;
    w = (max_seqlen_q > bm8 / 2 && wgs8 >= 192) ? 8 : 4;
  }
  const int bm = 32 * w / hpwg;            // query tokens per workgroup

  PrefillParams p;
  p.q = q;
  p.q_stride = q_token_stride;
  p.k = (const uint8_t*)k_cache;
  p.v = (const uint8_t*)v_cache;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.block_tables = block_tables;
  p.bt_stride = block_tables ? bt_stride : 0;
  p.kv_token_stride = kv_token_stride;
  p.cu_q = cu_seqlens_q;
  p.cu_k = cu_seqlens_k;
  p.out = out;
  p.out_stride = out_token_stride;
  p.q_dtype = q_dtype;
  p.num_q_heads = (int)num_q_heads;
  p.num_kv_heads = (int)num_kv_heads;
  p.bs_log2 = bs_log2;
  p.num_blocks = (int)num_blocks;
  p.scale_log2e = scale * 1.4426950408889634f;

  dim3 grid((unsigned)(num_q_heads / hpwg), (unsigned)((max_seqlen_q + bm - 1) / bm), (unsigned)num_seqs);
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (head_dim == 128)
    rc = w == 8 ? launch_prefill_hpwg<128, 8>(p, grid, hpwg, src, st) : launch_prefill_hpwg<128, 4>(p, grid, hpwg, src, st);
  else
    rc = w == 8 ? launch_prefill_hpwg<64, 8>(p, grid, hpwg, src, st) : launch_prefill_hpwg<64, 4>(p, grid, hpwg, src, st);
  if (rc != PA_OK) return rc;
  return check_launch("pa_prefill");
}
