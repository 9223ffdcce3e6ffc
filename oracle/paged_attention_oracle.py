"""CPU restatement of the reference's own PyTorch paged attention (the parity oracle).

TEST INFRASTRUCTURE ONLY.  Nothing under the product package imports this module; only
tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py do, and only as the
checker or as the timed CPU baseline.  It follows, function by function, the reference's
fallback path in src/inference/attention.py (the path that runs without flash-attn):

  store_kv_cache            attention.py:44-72    dispatcher
  store_kv_cache_fp16       attention.py:119-135  scatter copy, negative slots skipped
  store_kv_cache_fp8        attention.py:75-116   per-token 448/amax quantisation
  decode                    attention.py:317-382  per-sequence gather + SDPA
  decode_partitioned        attention.py:434-476  partition loop
  partition_attention       attention.py:519-589  local softmax, returns (out, lse)
  merge_partitions          attention.py:591-626  log-sum-exp merge
  prefill_no_prefix         attention.py:281-315  per-sequence causal SDPA on the new tokens
  prefill_paged             attention.py:240-257  flash_attn_varlen_func(causal, block_table)

Pinning (what fixes each function other than a retyped formula; see tests/test_oracle_*.py):
  * stores: closed form of a scatter, untouched-slot invariant, brute force per token;
    the e4m3fn cast against oracle/e4m3fn.py (an independent bit-level encoder) over every
    fp16 bit pattern and against known-answer bytes in tests/golden/e4m3fn_kat.json.
  * decode: fp64 brute force softmax(q.K^T).V on tiny inputs, ctx=1 returns V[0], block
    permutation invariance, garbage beyond the table invariance, GQA head map.
  * partitioned: merge == single pass, one partition == identity, lse == log(sum(exp)).
  * prefill_paged: the reference delegates this to flash-attn (un-vendored dependency
    `flash-attn>=2.5.0`, pyproject.toml:25), whose published semantics for causal=True with
    seqlen_q < seqlen_k is the bottom-right aligned mask; pinned by "row i == decode at
    context_len = cached + i + 1" and, without a prefix, by prefill_no_prefix.
  The reference holds no golden vectors or tests for this path, so none can be replayed.

Two reference quirks are made explicit instead of reproduced as failures:
  * the fp8 dequant `ki.to(float16) / scale` promotes K/V to fp32, and SDPA then rejects an
    fp16/bf16 query; the oracle upcasts q to fp32 for fp8 caches and casts the result back.
  * a bf16 query against an fp16 cache also raises in the reference; the oracle computes
    that case in fp32 and casts back.
"""
import math

import torch
import torch.nn.functional as F

FP8_DTYPE = torch.float8_e4m3fn
FP8_MAX = 448.0


# ---------------------------------------------------------------- KV cache write

def store_kv_cache_fp16(key, value, k_cache, v_cache, slot_mapping):
    """attention.py:119-135: rows of tokens with slot >= 0 are copied into the flat slot view."""
    num_blocks, block_size, num_kv_heads, head_dim = k_cache.shape
    total_slots = num_blocks * block_size
    k_flat = k_cache.view(total_slots, num_kv_heads, head_dim)
    v_flat = v_cache.view(total_slots, num_kv_heads, head_dim)
    valid = slot_mapping >= 0
    slots = slot_mapping[valid].long()
    k_flat[slots] = key[valid]
    v_flat[slots] = value[valid]


def quantize_fp8_per_token(x):
    """attention.py:101-110: amax over (heads, dim) in fp32, clamp 1e-5, s = 448/amax,
    bytes = (fp32(x) * s).to(e4m3fn).  Returns (fp8 tensor, fp32 scale [N]).

    `448.0 / amax` is a python float over a tensor, which torch evaluates as
    amax.reciprocal() * 448.0 (Tensor.__rtruediv__): two fp32 roundings, not one divide.  The
    expression is kept in the reference's form so that it follows torch, and
    tests/test_oracle_fp8.py pins the two-rounding closed form against numpy."""
    amax = x.float().abs().amax(dim=(-2, -1)).clamp(min=1e-5)
    s = FP8_MAX / amax
    q = (x.float() * s[:, None, None]).to(FP8_DTYPE)
    return q, s


def store_kv_cache_fp8(key, value, k_cache, v_cache, slot_mapping, k_scale, v_scale):
    """attention.py:75-116."""
    num_blocks, block_size, num_kv_heads, head_dim = k_cache.shape
    total_slots = num_blocks * block_size
    k_flat = k_cache.view(total_slots, num_kv_heads, head_dim)
    v_flat = v_cache.view(total_slots, num_kv_heads, head_dim)
    ks_flat = k_scale.view(total_slots)
    vs_flat = v_scale.view(total_slots)
    valid = slot_mapping >= 0
    slots = slot_mapping[valid].long()
    kq, ks = quantize_fp8_per_token(key[valid])
    vq, vs = quantize_fp8_per_token(value[valid])
    k_flat[slots] = kq
    v_flat[slots] = vq
    ks_flat[slots] = ks
    vs_flat[slots] = vs


def store_kv_cache(key, value, k_cache, v_cache, slot_mapping, k_scale=None, v_scale=None,
                   cache_dtype="fp16"):
    """attention.py:44-72 (the Triton branch is the same copy as the torch one)."""
    if cache_dtype == "fp8":
        store_kv_cache_fp8(key, value, k_cache, v_cache, slot_mapping, k_scale, v_scale)
    else:
        store_kv_cache_fp16(key, value, k_cache, v_cache, slot_mapping)


# ---------------------------------------------------------------- gather helpers

def _flat_indices(blocks, start, end, block_size):
    """attention.py:341-346 / 541-545: token positions -> flat physical slots."""
    pos = torch.arange(start, end)
    phys = blocks[pos // block_size]
    return phys.long() * block_size + pos % block_size


def _gather_kv(k_cache, v_cache, flat, k_scale, v_scale, fp8):
    """attention.py:349-362: gather, then fp8 -> fp16 -> divide by the per-token scale (fp32)."""
    num_kv_heads, head_dim = k_cache.shape[2], k_cache.shape[3]
    ki = k_cache.view(-1, num_kv_heads, head_dim)[flat]
    vi = v_cache.view(-1, num_kv_heads, head_dim)[flat]
    if fp8:
        ks = k_scale.view(-1)[flat]
        vs = v_scale.view(-1)[flat]
        ki = ki.to(torch.float16) / ks[:, None, None]
        vi = vi.to(torch.float16) / vs[:, None, None]
    return ki, vi


def _compute_dtype(q, kv_dtype, fp8):
    """dtype the reference's SDPA call would need; fp32 where the reference itself raises."""
    if fp8:
        return torch.float32
    if q.dtype != kv_dtype:
        return torch.float32
    return q.dtype


# ---------------------------------------------------------------- decode

def decode(q, k_cache, v_cache, block_tables, context_lens, scale, k_scale=None, v_scale=None,
           cache_dtype="fp16"):
    """attention.py:317-382.  q [B, Hq, D] -> [B, Hq, D] in q's dtype."""
    fp8 = cache_dtype == "fp8" and k_scale is not None
    num_blocks, block_size, num_kv_heads, head_dim = k_cache.shape
    num_heads = q.shape[1]
    cdt = _compute_dtype(q, k_cache.dtype, fp8)
    outs = []
    for i in range(q.shape[0]):
        ctx_len = int(context_lens[i])
        if ctx_len <= 0:
            # padded graph row: the reference would feed SDPA an empty key set (NaN); the
            # documented contract here is a zero row
            outs.append(torch.zeros_like(q[i:i + 1]))
            continue
        flat = _flat_indices(block_tables[i], 0, ctx_len, block_size)
        ki, vi = _gather_kv(k_cache, v_cache, flat, k_scale, v_scale, fp8)
        qi = q[i:i + 1].to(cdt)
        ki, vi = ki.to(cdt), vi.to(cdt)
        if num_kv_heads < num_heads:
            rep = num_heads // num_kv_heads
            ki = ki.repeat_interleave(rep, dim=1)
            vi = vi.repeat_interleave(rep, dim=1)
        oi = F.scaled_dot_product_attention(qi.transpose(0, 1), ki.transpose(0, 1),
                                            vi.transpose(0, 1), is_causal=False, scale=scale)
        outs.append(oi.transpose(0, 1).to(q.dtype))
    return torch.cat(outs, dim=0)


# ---------------------------------------------------------------- partitioned decode

def partition_attention(qi, k_cache, v_cache, blocks, start, end, block_size, scale,
                        k_scale=None, v_scale=None, fp8=False):
    """attention.py:519-589: attention over tokens [start, end) -> (out [1,H,D], lse [1,H])."""
    num_kv_heads = k_cache.shape[2]
    num_heads = qi.shape[1]
    flat = _flat_indices(blocks, start, end, block_size)
    ki, vi = _gather_kv(k_cache, v_cache, flat, k_scale, v_scale, fp8)
    ki, vi = ki.to(qi.dtype), vi.to(qi.dtype)
    if num_kv_heads < num_heads:
        rep = num_heads // num_kv_heads
        ki = ki.repeat_interleave(rep, dim=1)
        vi = vi.repeat_interleave(rep, dim=1)
    qh = qi.squeeze(0)                                   # [H, D]
    scores = torch.matmul(qh.unsqueeze(1), ki.permute(1, 2, 0)).squeeze(1) * scale  # [H, len]
    lse = torch.logsumexp(scores, dim=-1)
    w = torch.softmax(scores, dim=-1)
    out = torch.matmul(w.unsqueeze(1), vi.transpose(0, 1)).squeeze(1)              # [H, D]
    return out.unsqueeze(0), lse.unsqueeze(0)


def merge_partitions(partition_outputs, partition_lse):
    """attention.py:591-626."""
    lse = torch.cat(partition_lse, dim=0)                       # [P, H]
    g = torch.logsumexp(lse, dim=0)                             # [H]
    w = torch.exp(lse - g.unsqueeze(0))                         # [P, H]
    outs = torch.cat(partition_outputs, dim=0)                  # [P, H, D]
    return (outs * w.unsqueeze(-1)).sum(dim=0, keepdim=True)


def decode_partitioned(q, k_cache, v_cache, block_tables, context_lens, scale, partition_size=512,
                       k_scale=None, v_scale=None, cache_dtype="fp16", compute_dtype=None):
    """attention.py:434-476.  Sequences no longer than one partition take the plain decode.

    compute_dtype: dtype of the partition arithmetic.  The reference uses q's dtype (fp16
    scores and merge on CPU); pass torch.float32 to remove that rounding from a comparison.
    """
    fp8 = cache_dtype == "fp8" and k_scale is not None
    block_size = k_cache.shape[1]
    cdt = compute_dtype or _compute_dtype(q, k_cache.dtype, fp8)
    outs = []
    for i in range(q.shape[0]):
        ctx_len = int(context_lens[i])
        if ctx_len <= partition_size:
            outs.append(decode(q[i:i + 1], k_cache, v_cache, block_tables[i:i + 1],
                               context_lens[i:i + 1], scale, k_scale, v_scale, cache_dtype))
            continue
        qi = q[i:i + 1].to(cdt)
        n_part = (ctx_len + partition_size - 1) // partition_size
        p_out, p_lse = [], []
        for p in range(n_part):
            start = p * partition_size
            end = min(start + partition_size, ctx_len)
            o, l = partition_attention(qi, k_cache, v_cache, block_tables[i], start, end,
                                       block_size, scale, k_scale, v_scale, fp8)
            p_out.append(o)
            p_lse.append(l)
        outs.append(merge_partitions(p_out, p_lse).to(q.dtype))
    return torch.cat(outs, dim=0)


# ---------------------------------------------------------------- prefill

def prefill_no_prefix(q, k, v, cu_seqlens_q, cu_seqlens_k, scale):
    """attention.py:281-315: per-sequence causal SDPA over the new tokens (Lq == Lk)."""
    num_heads, num_kv_heads = q.shape[1], k.shape[1]
    outs = []
    for i in range(len(cu_seqlens_q) - 1):
        qs, qe = int(cu_seqlens_q[i]), int(cu_seqlens_q[i + 1])
        ks, ke = int(cu_seqlens_k[i]), int(cu_seqlens_k[i + 1])
        qi, ki, vi = q[qs:qe], k[ks:ke], v[ks:ke]
        if num_kv_heads < num_heads:
            rep = num_heads // num_kv_heads
            ki = ki.repeat_interleave(rep, dim=1)
            vi = vi.repeat_interleave(rep, dim=1)
        oi = F.scaled_dot_product_attention(qi.transpose(0, 1), ki.transpose(0, 1),
                                            vi.transpose(0, 1), is_causal=True, scale=scale)
        outs.append(oi.transpose(0, 1))
    return torch.cat(outs, dim=0)


def prefill_paged(q, k_cache, v_cache, block_tables, cu_seqlens_q, cu_seqlens_k, scale,
                  k_scale=None, v_scale=None, cache_dtype="fp16"):
    """attention.py:243-257 with block_tables set: K/V come from the paged cache, and row i of a
    sequence's chunk sees keys [0, Lk - Lq + i] (flash-attn's bottom-right causal alignment).
    Computed in fp32 (bf16 q against an fp16 cache has no common dtype), cast back to q's."""
    fp8 = cache_dtype == "fp8" and k_scale is not None
    block_size = k_cache.shape[1]
    num_heads, num_kv_heads = q.shape[1], k_cache.shape[2]
    outs = []
    for i in range(len(cu_seqlens_q) - 1):
        qs, qe = int(cu_seqlens_q[i]), int(cu_seqlens_q[i + 1])
        lk = int(cu_seqlens_k[i + 1]) - int(cu_seqlens_k[i])
        lq = qe - qs
        if lq == 0:
            continue
        flat = _flat_indices(block_tables[i], 0, lk, block_size)
        ki, vi = _gather_kv(k_cache, v_cache, flat, k_scale, v_scale, fp8)
        qi, ki, vi = q[qs:qe].float(), ki.float(), vi.float()
        if num_kv_heads < num_heads:
            rep = num_heads // num_kv_heads
            ki = ki.repeat_interleave(rep, dim=1)
            vi = vi.repeat_interleave(rep, dim=1)
        rows = torch.arange(lq)[:, None]
        cols = torch.arange(lk)[None, :]
        mask = cols <= rows + (lk - lq)
        oi = F.scaled_dot_product_attention(qi.transpose(0, 1), ki.transpose(0, 1),
                                            vi.transpose(0, 1), attn_mask=mask, scale=scale)
        outs.append(oi.transpose(0, 1).to(q.dtype))
    return torch.cat(outs, dim=0)


# ---------------------------------------------------------------- fp64 closed form (pins the above)

def decode_f64(q, k_cache, v_cache, block_tables, context_lens, scale, k_scale=None,
               v_scale=None):
    """softmax(scale * q.K^T).V written out in fp64 with explicit Python loops over sequences
    and heads; shares no code with decode() beyond torch indexing."""
    num_blocks, block_size, num_kv_heads, head_dim = k_cache.shape
    B, H, D = q.shape
    G = H // num_kv_heads
    out = torch.zeros(B, H, D, dtype=torch.float64)
    kf = k_cache.to(torch.float32).double().reshape(num_blocks * block_size, num_kv_heads, head_dim)
    vf = v_cache.to(torch.float32).double().reshape(num_blocks * block_size, num_kv_heads, head_dim)
    if k_scale is not None:
        kf = kf / k_scale.reshape(-1).double()[:, None, None]
        vf = vf / v_scale.reshape(-1).double()[:, None, None]
    for b in range(B):
        n = int(context_lens[b])
        if n <= 0:
            continue
        slots = [int(block_tables[b, t // block_size]) * block_size + t % block_size for t in range(n)]
        for h in range(H):
            K = kf[slots, h // G]                          # [n, D]
            V = vf[slots, h // G]
            s = (K @ q[b, h].double()) * scale
            s = s - s.max()
            p = torch.exp(s)
            out[b, h] = (p[:, None] * V).sum(0) / p.sum()
    return out
