"""Paged attention ops and modules backed by the gfx950 HIP kernels.

Same names, argument order and defaults as the reference's src/inference/attention.py
(store_kv_cache :44-72, PagedAttention :188-382, PartitionedPagedAttention :387-626), so a model
runner that binds caches by isinstance() and sets the global context can use these classes
unchanged.  Everything computes on the GPU through libpaged_attn.so; a CPU tensor or a
missing library raises RuntimeError (there is no fallback path).
"""
import contextlib
import functools
import os
from typing import Optional

import torch
import torch.nn as nn

from . import _native
from .context import get_context
from .kv_cache import HAS_FP8, _FP8_DTYPE

# Probe flags kept for callers that import them from the reference module.  Neither
# flash-attn nor Triton is used here.
HAS_FLASH_ATTN = False
HAS_TRITON = False

_DTYPE_CODE = {
    torch.float16: _native.DTYPE_F16,
    torch.bfloat16: _native.DTYPE_BF16,
    torch.float32: _native.DTYPE_F32,
}
if HAS_FP8:
    _DTYPE_CODE[_FP8_DTYPE] = _native.DTYPE_FP8_E4M3


def _code(dtype, what):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError("%s: unsupported dtype %s" % (what, dtype)) from None


def _require_gpu(t, what):
    if not t.is_cuda:
        raise RuntimeError(
            "%s: tensor is on %s; the paged-attention kernels run on the GPU only and this "
            "package has no CPU path" % (what, t.device))


# The current stream's handle without building a torch.cuda.Stream object around it: this runs once per
# kernel launch, and an eager decode step makes 140 of them.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(device):
    idx = device if isinstance(device, int) else device.index
    if idx is None:
        idx = torch.cuda.current_device()
    if _raw_stream is not None:
        return _raw_stream(idx)
    return torch.cuda.current_stream(idx).cuda_stream


def _rows(t, what):
    """[N, H, D] tensor with contiguous (H, D) -> (tensor, token stride in elements)."""
    if t.dim() != 3:
        raise RuntimeError("%s: expected [tokens, heads, head_dim], got %s" % (what, tuple(t.shape)))
    if t.stride(2) != 1 or t.stride(1) != t.shape[2] or (t.shape[0] > 1 and t.stride(0) < t.shape[1] * t.shape[2]):
        t = t.contiguous()
    return t, (t.stride(0) if t.shape[0] > 1 else t.shape[1] * t.shape[2])


def _int32(t, what):
    if t.dtype != torch.int32:
        t = t.to(torch.int32)
    if not t.is_contiguous():
        t = t.contiguous()
    return t


def _check_cache(k_cache, v_cache, what):
    if k_cache.dim() != 4 or v_cache.shape != k_cache.shape:
        raise RuntimeError("%s: caches must both be [num_blocks, block_size, kv_heads, head_dim]" % what)
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise RuntimeError("%s: cache layer views must be contiguous" % what)
    if k_cache.dtype != v_cache.dtype:
        raise RuntimeError("%s: k_cache and v_cache dtypes differ" % what)


# ==================== KV cache write ====================

def store_kv_cache(
    key: torch.Tensor,
    value: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    k_scale: Optional[torch.Tensor] = None,
    v_scale: Optional[torch.Tensor] = None,
    cache_dtype: str = "fp16",
):
    """Write new K/V rows into their physical cache slots.

    key, value   [num_tokens, num_kv_heads, head_dim]
    k_cache/v_cache  [num_blocks, block_size, num_kv_heads, head_dim] (one layer)
    slot_mapping [num_tokens] int32, slot = block_id * block_size + offset, negative = skip
    k_scale/v_scale  [num_blocks, block_size] fp32, fp8 mode only
    cache_dtype  "fp16" (bit copy in the cache dtype) or "fp8" (per-token 448/amax quantisation)

    Dispatch follows src/inference/attention.py:67-72: fp8 when requested and available,
    otherwise the copy.
    """
    _require_gpu(key, "store_kv_cache")
    _require_gpu(k_cache, "store_kv_cache")
    _check_cache(k_cache, v_cache, "store_kv_cache")
    lib = _native.load()
    num_blocks, block_size, num_kv_heads, head_dim = k_cache.shape
    total_slots = num_blocks * block_size
    row = num_kv_heads * head_dim
    n = key.shape[0]
    if value.shape != key.shape or tuple(key.shape[1:]) != (num_kv_heads, head_dim):
        raise RuntimeError("store_kv_cache: key/value shape %s/%s does not match the cache %s"
                           % (tuple(key.shape), tuple(value.shape), tuple(k_cache.shape)))
    if slot_mapping.numel() != n:
        raise RuntimeError("store_kv_cache: slot_mapping has %d entries for %d tokens"
                           % (slot_mapping.numel(), n))
    if n == 0:
        return
    key, ks = _rows(key, "store_kv_cache")
    value, vs = _rows(value, "store_kv_cache")
    slots = _int32(slot_mapping, "store_kv_cache")
    stream = _stream_ptr(key.device)

    if cache_dtype == "fp8" and HAS_FP8:
        if k_cache.dtype != _FP8_DTYPE:
            raise RuntimeError("store_kv_cache: cache_dtype='fp8' needs float8_e4m3fn caches, got %s"
                               % k_cache.dtype)
        if k_scale is None or v_scale is None:
            raise RuntimeError("store_kv_cache: fp8 mode needs k_scale and v_scale")
        if (k_scale.numel() != total_slots or v_scale.numel() != total_slots
                or k_scale.dtype != torch.float32 or v_scale.dtype != torch.float32
                or not k_scale.is_contiguous() or not v_scale.is_contiguous()):
            raise RuntimeError("store_kv_cache: scales must be contiguous fp32 [num_blocks, block_size]")
        if value.dtype != key.dtype:
            raise RuntimeError("store_kv_cache: key and value dtypes differ")
        rc = lib.pa_kv_store_fp8(key.data_ptr(), value.data_ptr(), _code(key.dtype, "store_kv_cache"),
                                 ks, vs, k_cache.data_ptr(), v_cache.data_ptr(),
                                 k_scale.data_ptr(), v_scale.data_ptr(), slots.data_ptr(), n, row,
                                 total_slots, stream)
        _native.check(rc, "pa_kv_store_fp8")
    else:
        if key.dtype != k_cache.dtype or value.dtype != v_cache.dtype:
            # the reference's index_put_ refuses mixed dtypes as well
            raise RuntimeError("store_kv_cache: key/value dtype %s does not match the cache dtype %s"
                               % (key.dtype, k_cache.dtype))
        rc = lib.pa_kv_store(key.data_ptr(), value.data_ptr(), ks, vs, k_cache.data_ptr(),
                             v_cache.data_ptr(), slots.data_ptr(), n, row, key.element_size(),
                             total_slots, stream)
        _native.check(rc, "pa_kv_store")


# ==================== decode launcher ====================

_WORKSPACES = {}


def qk_norm_rope_store(q, k, v, q_norm_weight, k_norm_weight, eps, inv_freq, positions,
                       k_cache=None, v_cache=None, slot_mapping=None, k_scale=None, v_scale=None,
                       cache_dtype="fp16", return_k=False):
    """Per-head RMSNorm of q and k, rotary embedding of both, and the paged cache write of k and
    v in one launch: what a Qwen3 attention block does between its projections and the
    attention call (src/distributed/tensor_parallel.py:78-84, 394-419, 453-464) followed by
    store_kv_cache (src/inference/attention.py:44-183).

    q [T, Hq, D], k / v [T, Hkv, D] (views with a token stride are fine), weights [D],
    inv_freq fp32 [D/2], positions int64 [T].  Returns (q_out, k_out) with k_out None unless
    return_k.  Without caches (or without a slot_mapping) nothing is written to the pool.
    """
    _require_gpu(q, "qk_norm_rope_store")
    lib = _native.load()
    if q.dim() != 3 or k.dim() != 3 or q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2]:
        raise RuntimeError("qk_norm_rope_store: expected q [T,Hq,D] and k [T,Hkv,D], got %s and %s"
                           % (tuple(q.shape), tuple(k.shape)))
    n, hq, d = q.shape
    hkv = k.shape[1]
    if k.dtype != q.dtype or (v is not None and v.dtype != q.dtype):
        raise RuntimeError("qk_norm_rope_store: q, k and v dtypes differ")
    def rows16(t):
        """rows as the kernel moves them: 16-byte pieces"""
        t, stride = _rows(t, "qk_norm_rope_store")
        if t.data_ptr() % 16 or (stride * t.element_size()) % 16:
            t = t.contiguous()
            stride = t.shape[1] * t.shape[2]
        return t, stride
    q, qs = rows16(q)
    k, ks_ = rows16(k)
    if q_norm_weight.numel() != d or k_norm_weight.numel() != d or q_norm_weight.dtype != k_norm_weight.dtype:
        raise RuntimeError("qk_norm_rope_store: norm weights must both be [head_dim] of one dtype")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() != d // 2:
        raise RuntimeError("qk_norm_rope_store: inv_freq must be fp32 [head_dim / 2]")
    if positions.numel() != n:
        raise RuntimeError("qk_norm_rope_store: positions has %d entries for %d tokens" % (positions.numel(), n))
    if positions.dtype != torch.int64 or not positions.is_contiguous():
        positions = positions.to(torch.int64).contiguous()
    q_out = torch.empty((n, hq, d), dtype=q.dtype, device=q.device)
    k_out = torch.empty((n, hkv, d), dtype=q.dtype, device=q.device) if return_k else None
    write = k_cache is not None and slot_mapping is not None
    vs_ = 0
    kv_code = _code(q.dtype, "qk_norm_rope_store")
    total_slots = 0
    if write:
        _check_cache(k_cache, v_cache, "qk_norm_rope_store")
        if tuple(k_cache.shape[2:]) != (hkv, d) or v is None or v.shape != k.shape:
            raise RuntimeError("qk_norm_rope_store: k/v %s do not match the cache %s"
                               % (tuple(k.shape), tuple(k_cache.shape)))
        v, vs_ = rows16(v)
        total_slots = k_cache.shape[0] * k_cache.shape[1]
        if slot_mapping.numel() != n:
            raise RuntimeError("qk_norm_rope_store: slot_mapping has %d entries for %d tokens"
                               % (slot_mapping.numel(), n))
        slot_mapping = _int32(slot_mapping, "qk_norm_rope_store")
        if cache_dtype == "fp8" and HAS_FP8:
            if k_cache.dtype != _FP8_DTYPE or k_scale is None or v_scale is None:
                raise RuntimeError("qk_norm_rope_store: cache_dtype='fp8' needs float8_e4m3fn caches and scales")
            kv_code = _native.DTYPE_FP8_E4M3
        elif k_cache.dtype != q.dtype:
            raise RuntimeError("qk_norm_rope_store: cache dtype %s differs from the activations' %s"
                               % (k_cache.dtype, q.dtype))
    if n == 0:
        return q_out, k_out
    fp8 = kv_code == _native.DTYPE_FP8_E4M3
    rc = lib.pa_qk_norm_rope_store(
        q.data_ptr(), k.data_ptr(), v.data_ptr() if write else None, _code(q.dtype, "qk_norm_rope_store"),
        qs, ks_, vs_, q_norm_weight.data_ptr(), k_norm_weight.data_ptr(),
        _code(q_norm_weight.dtype, "qk_norm_rope_store"), float(eps), inv_freq.data_ptr(), positions.data_ptr(),
        q_out.data_ptr(), hq * d, k_out.data_ptr() if return_k else None, hkv * d,
        k_cache.data_ptr() if write else None, v_cache.data_ptr() if write else None,
        k_scale.data_ptr() if (write and fp8) else None, v_scale.data_ptr() if (write and fp8) else None,
        kv_code, slot_mapping.data_ptr() if write else None, n, hq, hkv, d, total_slots, _stream_ptr(q.device))
    if rc != 0:
        raise RuntimeError("pa_qk_norm_rope_store failed (%d): %s"
                           % (rc, lib.pa_last_error().decode("utf-8", "replace")))
    return q_out, k_out


def sample_tokens(logits, temperature=0.7, top_p=0.9, uniforms=None, generator=None):
    """One token id per row of logits [batch, vocab] -> int64 [batch] on the same device, without
    a sort and without synchronising with the host (src/inference/model_runner.py:590-634).
    temperature <= 0 is greedy.  uniforms: fp32 [batch] in [0, 1) for a reproducible draw; by
    default drawn here from `generator` (or the device's default generator)."""
    _require_gpu(logits, "sample_tokens")
    if logits.dim() != 2:
        raise RuntimeError("sample_tokens: expected [batch, vocab], got %s" % (tuple(logits.shape),))
    lib = _native.load()
    if logits.stride(1) != 1:
        logits = logits.contiguous()
    b, vocab = logits.shape
    out = torch.empty(b, dtype=torch.int64, device=logits.device)
    if b == 0:
        return out
    if temperature > 0:
        if uniforms is None:
            uniforms = torch.rand(b, device=logits.device, dtype=torch.float32, generator=generator)
        if uniforms.numel() != b or uniforms.dtype != torch.float32 or not uniforms.is_cuda:
            raise RuntimeError("sample_tokens: uniforms must be fp32 [batch] on the GPU")
        uniforms = uniforms.contiguous()
    rc = lib.pa_sample(logits.data_ptr(), _code(logits.dtype, "sample_tokens"), logits.stride(0) if b > 1 else vocab,
                       b, vocab, float(temperature), float(top_p),
                       uniforms.data_ptr() if temperature > 0 else None, out.data_ptr(), _stream_ptr(logits.device))
    if rc != 0:
        raise RuntimeError("pa_sample failed (%d): %s" % (rc, lib.pa_last_error().decode("utf-8", "replace")))
    return out


def gather_kv_cache(k_cache, v_cache, block_tables, context_lens, out_len, len_offset=1):
    """Dense, head-major copies of the paged K and V of a batch:
    (k, v) each [batch, kv_heads, out_len, head_dim] in the cache's own dtype, rows at or past
    context_lens - len_offset zero.  One layer of ModelRunner._load_kv_from_paged_cache
    (src/inference/model_runner.py:340-420) without its host loops."""
    _require_gpu(k_cache, "gather_kv_cache")
    _check_cache(k_cache, v_cache, "gather_kv_cache")
    lib = _native.load()
    num_blocks, block_size, num_kv_heads, head_dim = k_cache.shape
    if block_tables.dim() != 2 or context_lens.numel() != block_tables.shape[0]:
        raise RuntimeError("gather_kv_cache: block_tables [batch, max_blocks] and context_lens [batch] expected")
    tables = block_tables if block_tables.dtype == torch.int32 else block_tables.to(torch.int32)
    if tables.stride(1) != 1:
        tables = tables.contiguous()
    lens = _int32(context_lens, "gather_kv_cache")
    batch = tables.shape[0]
    k_out = torch.empty((batch, num_kv_heads, int(out_len), head_dim), dtype=k_cache.dtype, device=k_cache.device)
    v_out = torch.empty_like(k_out)
    rc = lib.pa_gather_kv(k_cache.data_ptr(), v_cache.data_ptr(), tables.data_ptr(), tables.stride(0), tables.shape[1],
                          lens.data_ptr(), int(len_offset), k_out.data_ptr(), v_out.data_ptr(), batch, num_kv_heads,
                          head_dim, k_cache.element_size(), block_size, num_blocks, int(out_len),
                          _stream_ptr(k_cache.device))
    _native.check(rc, "pa_gather_kv")
    return k_out, v_out


def _rows2d(t, what):
    """[rows, width] view whose rows are 16-byte aligned and unit-stride inside; (tensor, row stride)."""
    if t.dim() != 2:
        raise RuntimeError("%s: expected a 2-D tensor, got %s" % (what, tuple(t.shape)))
    es = t.element_size()
    if t.stride(1) != 1 or (t.stride(0) * es) % 16 != 0 or t.data_ptr() % 16 != 0:
        t = t.contiguous()
    return t, (t.stride(0) if t.shape[0] > 1 else t.shape[1])


def add_rms_norm(x, weight, eps=1e-6, delta=None, inplace_sum=True):
    """RMSNorm of the residual stream, fused with the residual add that precedes it
    (src/distributed/tensor_parallel.py:78-84 and :640-651).  x [rows, hidden]; with delta
    [rows, hidden] returns (x + delta, norm(x + delta)) - the sum is written into x when
    inplace_sum - and without it (x, norm(x)).  Same roundings as the separate ops."""
    _require_gpu(x, "add_rms_norm")
    lib = _native.load()
    shape = x.shape
    flat = len(shape) == 2          # the decoder block's own call: nothing to reshape on the way in or out
    x2, xs = _rows2d(x if flat else x.reshape(-1, shape[-1]), "add_rms_norm")
    rows, hidden = x2.shape
    code = _code(x2.dtype, "add_rms_norm")
    normed = torch.empty((rows, hidden), dtype=x2.dtype, device=x2.device)
    if weight.numel() != hidden or not weight.is_contiguous():
        raise RuntimeError("add_rms_norm: weight must be contiguous [hidden]")
    d2 = ds = None
    total = x2
    if delta is not None:
        if delta.shape != shape or delta.dtype != x.dtype:
            raise RuntimeError("add_rms_norm: delta must match x in shape and dtype")
        d2, ds = _rows2d(delta if flat else delta.reshape(-1, hidden), "add_rms_norm")
        total = x2 if inplace_sum else torch.empty((rows, hidden), dtype=x2.dtype, device=x2.device)
    rc = lib.pa_add_rms_norm(x2.data_ptr(), xs, d2.data_ptr() if d2 is not None else None, ds or 0,
                             weight.data_ptr(), _code(weight.dtype, "add_rms_norm"), float(eps),
                             total.data_ptr() if d2 is not None else None,
                             (total.stride(0) if rows > 1 else hidden) if d2 is not None else 0,
                             normed.data_ptr(), hidden, code, rows, hidden, _stream_ptr(x2.device))
    _native.check(rc, "pa_add_rms_norm")
    if flat:
        return total, normed
    return total.view(shape), normed.view(shape)


def silu_mul(gate, up=None):
    """silu(gate) * up of a SwiGLU MLP (src/distributed/tensor_parallel.py:295-299).  With one
    argument [rows, 2 * width] it is the packed gate|up projection output."""
    _require_gpu(gate, "silu_mul")
    lib = _native.load()
    if up is None:
        if gate.shape[-1] % 2:
            raise RuntimeError("silu_mul: packed gate|up needs an even width")
        width = gate.shape[-1] // 2
        packed, stride = _rows2d(gate.reshape(-1, 2 * width), "silu_mul")
        if (width * packed.element_size()) % 16 != 0:
            raise RuntimeError("silu_mul: width must be a multiple of 16 bytes")
        g, u, gs, us = packed, packed[:, width:], stride, stride
        lead = gate.shape[:-1]
    else:
        if up.shape != gate.shape or up.dtype != gate.dtype:
            raise RuntimeError("silu_mul: gate and up must match in shape and dtype")
        width = gate.shape[-1]
        g, gs = _rows2d(gate.reshape(-1, width), "silu_mul")
        u, us = _rows2d(up.reshape(-1, width), "silu_mul")
        lead = gate.shape[:-1]
    rows = g.shape[0]
    out = torch.empty((rows, width), dtype=g.dtype, device=g.device)
    rc = lib.pa_silu_mul(g.data_ptr(), gs, u.data_ptr(), us, out.data_ptr(), width, _code(g.dtype, "silu_mul"),
                         rows, width, _stream_ptr(g.device))
    _native.check(rc, "pa_silu_mul")
    return out.view(*lead, width)


def slot_mapping(positions, block_tables, block_size, num_blocks, cu_seqlens_q=None, out=None):
    """int32 [tokens] of physical cache slots, computed on the GPU without a host round trip:
    block_tables[row][position // block_size] * block_size + position % block_size.  Without
    cu_seqlens_q token i uses table row i (one new token per sequence, the loop at
    src/inference/model_runner.py:670-682); with it, row = the sequence whose chunk holds the
    token (model_runner.py:493-511).  Tokens whose position falls outside their table, or on a
    block id outside the pool (padding -1 included), get -1 and are skipped by the KV writers."""
    _require_gpu(positions, "slot_mapping")
    _require_gpu(block_tables, "slot_mapping")
    if block_tables.dim() != 2:
        raise RuntimeError("slot_mapping: block_tables must be [rows, max_blocks]")
    lib = _native.load()
    positions = positions.reshape(-1)
    if positions.dtype != torch.int64:
        positions = positions.to(torch.int64)
    positions = positions.contiguous()
    tables = block_tables if block_tables.dtype == torch.int32 else block_tables.to(torch.int32)
    if tables.stride(1) != 1:
        tables = tables.contiguous()
    n = positions.numel()
    if out is None:
        out = torch.empty(n, dtype=torch.int32, device=positions.device)
    elif out.dtype != torch.int32 or out.numel() != n or not out.is_contiguous():
        raise RuntimeError("slot_mapping: out must be contiguous int32 [tokens]")
    cu = None
    if cu_seqlens_q is not None:
        cu = _int32(cu_seqlens_q, "slot_mapping")
        if cu.numel() != tables.size(0) + 1:
            raise RuntimeError("slot_mapping: cu_seqlens_q must have rows + 1 entries")
    rc = lib.pa_slot_mapping(positions.data_ptr(), cu.data_ptr() if cu is not None else None, tables.data_ptr(),
                             tables.stride(0), out.data_ptr(), n, tables.size(0), tables.size(1), int(block_size),
                             int(num_blocks), _stream_ptr(positions.device))
    _native.check(rc, "pa_slot_mapping")
    return out


def prefill_metadata(cu_seqlens_q, cu_seqlens_k, num_tokens, block_tables=None, block_size=16, num_blocks=None,
                     row_index=None):
    """(positions int64 [num_tokens], slot_mapping int32 [num_tokens] or None) of a prefill step,
    computed on the GPU from its cumulative length arrays (src/inference/model_runner.py:479-511):
    token t of chunk r sits at position cached_r + t - cu_seqlens_q[r], and its slot comes from the
    sequence's row of block_tables (row_index[r] of a larger device-resident table when given, else
    row r).  Without block_tables only the positions are made."""
    _require_gpu(cu_seqlens_q, "prefill_metadata")
    lib = _native.load()
    cu_q = _int32(cu_seqlens_q, "prefill_metadata")
    cu_k = _int32(cu_seqlens_k, "prefill_metadata")
    num_seqs = cu_q.numel() - 1
    if cu_k.numel() != num_seqs + 1:
        raise RuntimeError("prefill_metadata: cu_seqlens_q and cu_seqlens_k differ in length")
    positions = torch.empty(int(num_tokens), dtype=torch.long, device=cu_q.device)
    slots = None
    bt_ptr, bt_stride, rows, width, idx_ptr = None, 0, 0, 0, None
    if block_tables is not None:
        if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or block_tables.stride(1) != 1:
            raise RuntimeError("prefill_metadata: block_tables must be int32 [rows, max_blocks] with unit column stride")
        if num_blocks is None:
            raise RuntimeError("prefill_metadata: num_blocks is needed with block_tables")
        slots = torch.empty(int(num_tokens), dtype=torch.int32, device=cu_q.device)
        bt_ptr, bt_stride, rows, width = block_tables.data_ptr(), block_tables.stride(0), block_tables.shape[0], block_tables.shape[1]
        if row_index is not None:
            row_index = _int32(row_index, "prefill_metadata")
            if row_index.numel() != num_seqs:
                raise RuntimeError("prefill_metadata: row_index must have one entry per sequence")
            idx_ptr = row_index.data_ptr()
        elif rows < num_seqs:
            raise RuntimeError("prefill_metadata: block_tables has %d rows for %d sequences" % (rows, num_seqs))
    rc = lib.pa_prefill_metadata(cu_q.data_ptr(), cu_k.data_ptr(), bt_ptr, bt_stride, idx_ptr, positions.data_ptr(),
                                 slots.data_ptr() if slots is not None else None, int(num_tokens), num_seqs, rows, width,
                                 int(block_size), int(num_blocks or 1), _stream_ptr(cu_q.device))
    _native.check(rc, "pa_prefill_metadata")
    return positions, slots


def _device_index(device):
    return device.index if device.index is not None else torch.cuda.current_device()


_GRAPHS = "graphs"
_sizing_for_graphs = 0


@contextlib.contextmanager
def sizing_graph_workspace():
    """While active, every partitioned decode launch also sizes the workspace that recorded graphs
    use, and launches are shaped as they will be inside the capture (the policy splits small launches
    differently for eager calls): wrap the warm-up runs that precede a capture in it."""
    global _sizing_for_graphs
    _sizing_for_graphs += 1
    try:
        yield
    finally:
        _sizing_for_graphs -= 1


def reserve_decode_workspace(device, nbytes, for_graphs=False):
    """Make a partition workspace at least `nbytes` large and return it.

    Workspaces are kept per (device, stream): launches that run at the same time on different
    streams of one GPU never share partials.  Launches recorded into a HIP graph use one more
    workspace per device, the graphs' own (for_graphs=True, and whenever the current stream is
    capturing): a capture runs on a side stream of its own, and the replays may run on any.  Graphs
    of one device share it, so two graphs replayed at the same time on different streams would
    race; give such launches their own tensor through paged_decode(workspace=...).
    A workspace only grows, and a tensor it has outgrown is kept alive, never handed back to the
    allocator: a recorded graph still holds that tensor's address.  Growing allocates, so it must
    happen outside a capture - whoever captures decode graphs reserves the largest size first
    (ModelRunner does, from its largest batch and the launch policy's partition limit; warm-up runs
    inside sizing_graph_workspace() do it too); inside a capture a workspace that is too small
    raises instead of allocating from the graph's pool."""
    idx = _device_index(device)
    capturing = _is_capturing()
    if _sizing_for_graphs and not capturing and not for_graphs:
        reserve_decode_workspace(device, nbytes, for_graphs=True)
    key = (idx, _GRAPHS if (for_graphs or capturing) else _stream_ptr(idx))
    held = _WORKSPACES.setdefault(key, [])
    if held and held[-1].numel() >= nbytes:
        return held[-1]
    if capturing:
        raise RuntimeError(
            "paged_decode: the graphs' partition workspace of cuda:%d holds %d bytes and this launch needs %d; "
            "it cannot grow during a graph capture - call reserve_decode_workspace(..., for_graphs=True) or run "
            "the warm-up inside sizing_graph_workspace() before capturing"
            % (idx, held[-1].numel() if held else 0, nbytes))
    ws = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=torch.device("cuda", idx))
    held.append(ws)
    return ws


def decode_workspace_bytes(batch, num_q_heads, head_dim, max_partitions=None):
    """Bytes of partition workspace that cover any launch of up to `batch` rows: by default for the
    finest split the launch policy ever chooses."""
    parts = _MAX_AUTO_PARTITIONS if max_partitions is None else int(max_partitions)
    return _native.load().pa_workspace_bytes(int(batch), int(num_q_heads), int(head_dim), parts)


def release_decode_workspaces():
    """Drop every partition workspace.  Only safe once no recorded graph that used one will be
    replayed again."""
    _WORKSPACES.clear()


def check_block_tables(block_tables, context_lens, block_size, num_blocks):
    """(entries outside the pool, rows whose context outruns the table), counted on the GPU over the
    part of each row that a decode launch would read.  The attention kernels clamp both instead of
    faulting, so a corrupt table shows up as wrong numbers; this is the check that names it.
    Synchronises with the host: a debugging aid (PA_DEBUG_TABLES=1 runs it before every decode)."""
    _require_gpu(block_tables, "check_block_tables")
    lib = _native.load()
    tables = block_tables if block_tables.dtype == torch.int32 else block_tables.to(torch.int32)
    if tables.stride(1) != 1:
        tables = tables.contiguous()
    lens = _int32(context_lens, "check_block_tables")
    counts = torch.zeros(2, dtype=torch.int32, device=tables.device)
    rc = lib.pa_check_tables(tables.data_ptr(), tables.stride(0), tables.shape[1], lens.data_ptr(),
                             tables.shape[0], int(block_size), int(num_blocks), counts.data_ptr(),
                             _stream_ptr(tables.device))
    _native.check(rc, "pa_check_tables")
    bad, short = counts.tolist()
    return bad, short


def _debug_tables():
    return os.environ.get("PA_DEBUG_TABLES", "0") not in ("", "0")


# ---- how a decode launch is shaped ------------------------------------------------------------
# Two rates bound a launch: what HBM delivers to the whole GPU, and what one CU can pull however
# many workgroups it hosts (about 1.3 x its 1/256 share).  Workgroups are dealt to CUs in rounds,
# so the launch lasts as long as its busiest CU needs: 288 equal workgroups on 256 CUs make two
# rounds, not 1.125.  The context is split where the larger of the two bounds, plus about 2 us per
# round of workgroups and 3 us + 0.03 us per partition for the merge pass, is smallest.  The rates
# are fitted to a sweep of every split on an MI355X (batch 1..128, contexts 2k..32k, fp16 and fp8
# caches, streaming loads): the pick is within 1.5 % of the best measured split on average, 7 % at worst.
_MIN_AUTO_PARTITION = 64           # tokens: the finest split (launches of a few rows: about one round of workgroups, however short)
_SINGLE_PASS_UP_TO = {2: 256, 1: 512}   # contexts (tokens) that are never split, by cache element size
_MIN_RAGGED_PARTITION = 384        # tokens
_MIN_RAGGED_BYTES = 96 << 20       # K and V bytes of a launch from which the split for ragged batches is used
_MAX_AUTO_PARTITIONS = 128
_HBM_BYTES_PER_NS = 6800.0
_CU_BYTES_PER_NS = {2: 28.0, 1: 25.0}      # by cache element size
_ROUND_NS = 2000.0
_MERGE_NS = (3000.0, 30.0)         # fixed, per partition (the pass itself and the partials it re-reads)
# An eager call (no graph) cannot return faster than the host can issue it: about 11.5 us for the call with
# one launch, 5 us more with the merge pass behind it.  Below that, what the split saves on the device is lost.
_EAGER_CALL_NS = (11500.0, 5000.0)
_EAGER_CHECK_TOKENS = 32768        # batch x context up to which an eager call looks at that
_LAUNCH_SHAPES = {}                # paged_decode's shapes -> what the policy said for them (replayed, eager)
_DEFAULT_COMPUTE_UNITS = 256
MATRIX_PATH_FROM_RATIO = 3         # GQA ratio from which pa_decode multiplies on the matrix cores (up to 16 query heads per workgroup)
_CU_COUNT = {}


_is_capturing = getattr(torch._C, "_cuda_isCurrentStreamCapturing", None) or torch.cuda.is_current_stream_capturing


def _compute_units(device):
    idx = device.index if device.index is not None else torch.cuda.current_device()
    n = _CU_COUNT.get(idx)
    if n is None:
        n = torch.cuda.get_device_properties(idx).multi_processor_count or _DEFAULT_COMPUTE_UNITS
        _CU_COUNT[idx] = n
    return n


def pairs_kv_heads(workgroups, can_pair, compute_units=_DEFAULT_COMPUTE_UNITS):
    """The launch's own rule (pa_decode) for serving two adjacent KV heads from one workgroup:
    when halving the `workgroups` of the unpaired launch does not add a round of them over the
    CUs (fewer, longer-lived workgroups stream better; with one workgroup or less per CU pairing
    would only idle CUs)."""
    if not can_pair:
        return False
    if workgroups >= 8 * compute_units:
        return True
    rounds = -(-workgroups // compute_units)
    paired_rounds = -(-workgroups // (2 * compute_units))
    return 2 * paired_rounds <= rounds


def _known_lengths(max_context, longest, mean):
    """The caller's knowledge of a batch's context lengths, brought into the form the policy caches on:
    the bound on the longest row rounded up to 256 tokens (never above the table's width), the mean as
    sixteenths of that bound (None = rows about as long as the bound: 11/16 of it or more)."""
    bound = int(max_context)
    if longest is not None and longest > 0:
        bound = min(bound, -(-int(longest) // 256) * 256)
    fill = None
    if mean is not None and mean > 0 and bound > 0:
        fill = max(1, min(16, int(round(16.0 * float(mean) / bound))))
        if fill >= 11:
            fill = None
    return bound, fill


@functools.lru_cache(maxsize=4096)
def _choose_partition(batch, num_q_heads, num_kv_heads, max_context, head_dim, kv_elem_bytes, compute_units,
                      mean_sixteenths, eager=False):
    if max_context <= _SINGLE_PASS_UP_TO.get(kv_elem_bytes, 256) or batch <= 0:
        return 0, 1
    g = num_q_heads // num_kv_heads
    if g >= MATRIX_PATH_FROM_RATIO:
        # the matrix kernel: one workgroup per KV head and slice of 16 query heads
        units = batch * num_kv_heads * -(-g // 16)
        can_pair = num_kv_heads % 2 == 0
    else:
        gc = 2 if g % 2 == 0 else 1
        can_pair = g == gc and num_kv_heads % 2 == 0
        units = batch * (num_q_heads // gc)              # workgroups of one partition, unpaired
    narrow = head_dim * kv_elem_bytes <= 128
    token_bytes = 2.0 * head_dim * kv_elem_bytes         # K and V of one head
    cu_rate = _CU_BYTES_PER_NS.get(kv_elem_bytes, 31.0)
    if mean_sixteenths is not None and \
            batch * num_kv_heads * (max_context * mean_sixteenths / 16.0) * token_bytes >= _MIN_RAGGED_BYTES:
        # A ragged batch (one large enough for the memory system to set the pace: below about 100 MB the
        # fixed costs of a launch do, and the split for full rows of the bound is the better one).  Partitions without tokens cost nothing (their workgroups are numbered last and
        # leave at once) and workgroups of unequal length do not march in rounds - a CU takes the next
        # one when it is done - so what counts is that there are enough of them to even out: about four
        # per CU.  Rows that provide that by themselves are read in one pass; otherwise the partition is
        # the largest (a multiple of 128 tokens, at least 384: finer ones lost to 384 in 11 of 12 measured
        # batches) that cuts the rows into that many pieces, a row of the mean length counting
        # mean / size whole partitions and half a one at its end.  Measured on an MI355X (4 to 256 rows,
        # lengths uniform between 1/16 and 1 of a bound of 512 to 16384 tokens, fp16 and fp8 caches):
        # up to 24 % faster than the split for full rows (never more than 2 % slower), within 12 % of the
        # best split of a sweep of sizes.
        mean_context = max_context * mean_sixteenths / 16.0
        single = units // 2 if pairs_kv_heads(units, can_pair, compute_units) else units
        want = 4 * compute_units
        if single >= want:
            return 0, 1
        paired = units // 2 if can_pair else units         # grids this large always pair
        psize = int(mean_context / (want / paired - 0.5)) // 128 * 128
        psize = max(_MIN_RAGGED_PARTITION, psize)
        parts = -(-max_context // psize)
        if parts > _MAX_AUTO_PARTITIONS:
            psize = -(-(-(-max_context // _MAX_AUTO_PARTITIONS)) // 128) * 128
            parts = -(-max_context // psize)
        return (0, 1) if parts <= 1 else (psize, parts)
    hbm_ns = batch * num_kv_heads * max_context * token_bytes / _HBM_BYTES_PER_NS
    best = None
    max_parts = max(1, min(_MAX_AUTO_PARTITIONS, max_context // _MIN_AUTO_PARTITION))
    seen = set()
    for want in range(1, max_parts + 1):
        psize = -(-max_context // want)
        psize = -(-psize // 16) * 16
        parts = -(-max_context // psize)
        if parts in seen:
            continue
        seen.add(parts)
        wgs = units * parts
        heads = 2 if pairs_kv_heads(wgs, can_pair, compute_units) else 1
        # lone rows of 128 bytes or less stream about 10% below the rest
        hbm = hbm_ns * (1.12 if narrow and heads == 1 else 1.0)
        rounds = -(-(wgs // heads) // compute_units)
        # a CU pulls more when most of the others have nothing to do: 8 workgroups stream at twice the
        # rate per CU that 256 do (measured at batch 1 to 32, contexts of 384 to 1024 tokens); from half
        # the CUs on the fitted rate stands
        lone = 1.0 + 0.8 * max(0.0, 1.0 - 2.0 * (wgs // heads) / float(compute_units))
        busiest_ns = rounds * min(psize, max_context) * heads * token_bytes / (cu_rate * lone)
        cost = max(hbm, busiest_ns) + rounds * _ROUND_NS
        if parts > 1:
            cost += _MERGE_NS[0] + _MERGE_NS[1] * parts
        if eager:
            cost = max(cost, _EAGER_CALL_NS[0] + (_EAGER_CALL_NS[1] if parts > 1 else 0.0))
        if best is None or cost < best[0] * 0.99:        # ties go to the coarser split
            best = (cost, psize, parts)
    _, psize, parts = best
    return (0, 1) if parts <= 1 else (psize, parts)


def choose_partition(batch, num_q_heads, num_kv_heads, max_context, head_dim=128, kv_elem_bytes=2,
                     compute_units=_DEFAULT_COMPUTE_UNITS, longest_context=None, mean_context=None, eager=False):
    """Partition size for a decode launch that has no caller-given one: the split of
    `max_context` (a multiple of 16 tokens, at least 64) with the smallest modelled time.
    Returns (partition_size, max_partitions); (0, 1) means a single pass.

    max_context is what the block table can hold.  A caller that knows its rows (the model runner has
    the lengths on the host) says so: longest_context bounds the rows, so the launch is sized for that
    instead of the table's width (a row beyond it is still computed exactly, its last partition runs
    to the row's end), and mean_context tells a ragged batch from a full one - a ragged one is split
    finer, because partitions without tokens cost nothing and the partitions with tokens spread evenly
    over the CUs where whole rows of unequal length do not.  eager: the launch is issued call by call,
    not replayed from a graph, so a split also costs the host a second launch (it is then only taken
    where the single pass would last longer than the two calls take to issue)."""
    bound, fill = _known_lengths(max_context, longest_context, mean_context)
    return _choose_partition(batch, num_q_heads, num_kv_heads, bound, head_dim, kv_elem_bytes, compute_units,
                             fill, bool(eager))


def choose_launch(batch, num_q_heads, num_kv_heads, max_context, head_dim=128, kv_elem_bytes=2,
                  compute_units=_DEFAULT_COMPUTE_UNITS, longest_context=None, mean_context=None, eager=False):
    """(partition_size, max_partitions, kv_heads_per_wave) of a decode launch that has no
    caller-given shape; kv_heads_per_wave 0 leaves the choice between one and two KV heads per
    wave to the launch itself (the rule of pairs_kv_heads)."""
    psize, parts = choose_partition(batch, num_q_heads, num_kv_heads, max_context, head_dim, kv_elem_bytes,
                                    compute_units, longest_context, mean_context, eager)
    return psize, parts, 0


# ---- shared prefixes ---------------------------------------------------------------------------
SHARED_PREFIX_PARTITION = 256      # tokens; the granularity at which a shared prefix is computed once


def find_prefix_groups(block_tables, context_lens, block_size, num_q_heads, num_kv_heads,
                       partition_size=SHARED_PREFIX_PARTITION):
    """Host-side: runs of consecutive rows whose leading table entries name the same physical
    blocks (n samples of a prompt, forks of a cached prefix), as [(first_row, rows, shared_tokens)].
    block_tables: per-row lists of block ids (what the cache manager holds on the host);
    context_lens: per-row token counts.  Only whole partitions count, a group needs two rows and
    one shared partition, and holds at most 16 // (num_q_heads // num_kv_heads) rows (the columns
    of the matrix kernel's operand); longer runs are cut into several groups, and a run ends where
    the next row would shrink what the group shares by more than it adds."""
    max_rows = 16 // max(1, num_q_heads // num_kv_heads)
    if max_rows < 2 or partition_size <= 0 or partition_size % block_size:
        return []
    part_blocks = partition_size // block_size
    groups, n, b = [], len(block_tables), 0
    while b < n:
        lead = block_tables[b]
        limit = min(len(lead), int(context_lens[b]) // block_size)     # whole blocks inside the context
        rows, shared = 1, limit
        while b + rows < n and rows < max_rows:
            other = block_tables[b + rows]
            cap = min(shared, len(other), int(context_lens[b + rows]) // block_size)
            common = 0
            while common < cap and other[common] == lead[common]:
                common += 1
            # a group of n rows saves n - 1 reads of its shared partitions: stop where taking the row
            # in would shrink the shared part by more than that adds
            new_parts, old_parts = common // part_blocks, shared // part_blocks
            if new_parts < 1 or (new_parts < old_parts and rows * new_parts <= (rows - 1) * old_parts):
                break
            shared = common
            rows += 1
        if rows >= 2:
            groups.append((b, rows, (shared // part_blocks) * partition_size))
        b += rows
    return groups


def _common_blocks(a, b, cap):
    """Leading entries, at most cap, that two block-id lists have in common (bisection over slice
    comparisons, which run at C speed)."""
    if a[:cap] == b[:cap]:
        return cap
    lo, hi = 0, cap                    # a[:lo] == b[:lo], a[:hi] != b[:hi]
    while hi - lo > 1:
        mid = (lo + hi) // 2
        if a[:mid] == b[:mid]:
            lo = mid
        else:
            hi = mid
    return lo


def find_prefix_groups_anywhere(block_tables, context_lens, block_size, num_q_heads, num_kv_heads,
                                partition_size=SHARED_PREFIX_PARTITION, rows=None):
    """find_prefix_groups for rows that share prefixes wherever they sit in the batch, as
    [([row, ...], shared_tokens)].  Rows that share anything share their first physical block, so
    the rows are bucketed by it (one dictionary pass; a batch without sharing costs nothing more).
    A bucket's rows are ordered by their block ids, which puts the longest common prefixes next to
    each other: what a run of the ordered rows shares is the smallest common prefix of its
    neighbours, and the cut of the order into runs of at most 16 // (num_q_heads // num_kv_heads)
    rows that saves the most reads ((rows - 1) x shared partitions per run) is found by dynamic
    programming.  rows: the batch rows the entries of block_tables belong to (default 0, 1, ...)."""
    max_rows = 16 // max(1, num_q_heads // num_kv_heads)
    if max_rows < 2 or partition_size <= 0 or partition_size % block_size:
        return []
    part_blocks = partition_size // block_size
    rows = list(range(len(block_tables))) if rows is None else list(rows)
    buckets = {}
    for i, table in enumerate(block_tables):
        if len(table) and int(context_lens[i]) >= partition_size:
            buckets.setdefault(table[0], []).append(i)
    out = []
    for members in buckets.values():
        n = len(members)
        if n < 2:
            continue
        members.sort(key=lambda i: block_tables[i])
        cap = [min(len(block_tables[i]), int(context_lens[i]) // block_size) for i in members]
        near = [_common_blocks(block_tables[members[k]], block_tables[members[k + 1]], min(cap[k], cap[k + 1]))
                for k in range(n - 1)]
        best = [0] * (n + 1)             # best[i]: most partition reads saved by cutting the first i rows
        cut = [None] * (n + 1)           # the last run of that cut as (start, shared blocks), None: row i - 1 alone
        for i in range(1, n + 1):
            best[i], cut[i] = best[i - 1], None
            shared = cap[i - 1]
            for j in range(i - 2, max(i - max_rows, 0) - 1, -1):      # the run members[j:i]
                shared = min(shared, near[j], cap[j])
                parts = shared // part_blocks
                if parts < 1:
                    break
                gain = best[j] + (i - j - 1) * parts
                if gain > best[i]:
                    best[i], cut[i] = gain, (j, shared)
        i = n
        while i > 0:
            if cut[i] is None:
                i -= 1
                continue
            j, shared = cut[i]
            out.append((sorted(rows[m] for m in members[j:i]), (shared // part_blocks) * partition_size))
            i = j
    out.sort(key=lambda g: g[0][0])
    return out


class PrefixGroups:
    """Device descriptors of a pa_decode_shared_prefix launch.

    group_desc int32 [capacity, 4] (first, rows, shared partitions, 0; groups past num_groups - and
    any group of 0 partitions - are empty), group_rows int32 [..] or None (None: a group's rows are
    consecutive batch rows from `first`; else they are group_rows[first : first + rows]), row_skip
    int32 [batch] (the leading partitions of a row that its group computes).  num_groups,
    max_group_rows, max_shared_partitions and min_row_skip are the host-side bounds the launch is
    sized with; a recorded graph fixes them at the descriptors' capacity."""

    def __init__(self, partition_size, group_desc, group_rows, row_skip, num_groups, max_group_rows,
                 max_shared_partitions, min_row_skip=0, groups=None):
        self.partition_size = int(partition_size)
        self.group_desc, self.group_rows, self.row_skip = group_desc, group_rows, row_skip
        self.num_groups, self.max_group_rows = int(num_groups), int(max_group_rows)
        self.max_shared_partitions, self.min_row_skip = int(max_shared_partitions), int(min_row_skip)
        self.groups = groups                   # host copy, for tests and debugging

    @property
    def batch(self):
        return self.row_skip.numel()


def _normalise_groups(groups):
    """[(first, rows, tokens)] or [([rows], tokens)] -> ([([rows], tokens)], all consecutive?)"""
    norm, consecutive = [], True
    for g in groups:
        if len(g) == 3:
            first, count, tokens = g
            norm.append((list(range(int(first), int(first) + int(count))), int(tokens)))
        else:
            members, tokens = g
            members = [int(r) for r in members]
            consecutive = consecutive and members == list(range(members[0], members[0] + len(members)))
            norm.append((members, int(tokens)))
    return norm, consecutive


def shared_prefix_descriptors(groups, batch, device, partition_size=SHARED_PREFIX_PARTITION):
    """PrefixGroups for [(first_row, rows, shared_tokens)] (find_prefix_groups) or
    [([row, ...], shared_tokens)] (find_prefix_groups_anywhere): one pinned host buffer, one copy."""
    norm, consecutive = _normalise_groups(groups)
    ng = len(norm)
    host = torch.zeros(4 * max(ng, 1) + 2 * batch, dtype=torch.int32)
    desc = host[:4 * max(ng, 1)].view(-1, 4)
    rows_flat = host[4 * max(ng, 1):4 * max(ng, 1) + batch]
    skip = host[4 * max(ng, 1) + batch:]
    max_rows = max_parts = cursor = 0
    for i, (members, shared_tokens) in enumerate(norm):
        parts = shared_tokens // partition_size
        if not members or min(members) < 0 or max(members) >= batch:
            raise RuntimeError("shared_prefix_descriptors: group %s reaches outside the batch of %d" % (members, batch))
        if cursor + len(members) > batch:
            raise RuntimeError("shared_prefix_descriptors: rows claimed by more than one group")
        desc[i, 0] = members[0] if consecutive else cursor
        desc[i, 1], desc[i, 2] = len(members), parts
        rows_flat[cursor:cursor + len(members)] = torch.tensor(members, dtype=torch.int32)
        cursor += len(members)
        skip[torch.tensor(members, dtype=torch.long)] = parts
        max_rows, max_parts = max(max_rows, len(members)), max(max_parts, parts)
    min_skip = int(skip.min()) if batch else 0
    dev = host.pin_memory().to(device, non_blocking=True) if torch.device(device).type == "cuda" else host
    n4 = 4 * max(ng, 1)
    return PrefixGroups(partition_size, dev[:n4].view(-1, 4), None if consecutive else dev[n4:n4 + batch],
                        dev[n4 + batch:], ng, max(1, max_rows), max_parts, min_skip, groups=norm)


def choose_prefix_partition(find, sizes=(2048, 1024, 512, 256), keep=0.9):
    """The coarsest partition size of `sizes` whose groups still keep `keep` of the reads that the
    finest size saves (coarser partitions mean fewer, longer-lived workgroups and fewer partials to
    merge: the fourth benchmark configuration takes 119 us at 256 tokens, 93 at 512, 87 at 1024).
    find(size) -> groups as the finders return them.  Returns (size, groups) or (None, [])."""
    def saved(groups):
        return sum((len(g[0]) - 1 if len(g) == 2 else g[1] - 1) * g[-1] for g in groups)
    sizes = sorted(sizes, reverse=True)
    fine = find(sizes[-1])
    if not fine:
        return None, []
    for size in sizes[:-1]:
        coarse = find(size)
        if coarse and saved(coarse) >= keep * saved(fine):
            return size, coarse
    return sizes[-1], fine


def prepare_prefix_groups(block_tables, context_lens, block_size, num_q_heads, num_kv_heads, device,
                          partition_size=None, anywhere=False):
    """What a decode step hands the attention layers (InferenceContext.prefix_groups) when rows share
    prefixes: the groups found on the host in the per-row block-id lists and their device descriptors
    (a PrefixGroups), built once per step for all layers.  None when no two rows share a whole
    partition.  partition_size None: choose_prefix_partition's pick.  anywhere: group rows wherever
    they sit in the batch (find_prefix_groups_anywhere) instead of runs of consecutive rows."""
    finder = find_prefix_groups_anywhere if anywhere else find_prefix_groups

    def find(size):
        if size % block_size:
            return []
        return finder(block_tables, context_lens, block_size, num_q_heads, num_kv_heads, size)

    if partition_size is None:
        partition_size, groups = choose_prefix_partition(find)
    else:
        groups = find(int(partition_size))
    if not groups:
        return None
    return shared_prefix_descriptors(groups, len(block_tables), device, partition_size)


def paged_decode_shared_prefix(q, k_cache, v_cache, block_tables, context_lens, scale, groups, k_scale=None,
                               v_scale=None, partition_size=SHARED_PREFIX_PARTITION, out=None, waves=0,
                               workspace=None, descriptors=None, longest_context=None):
    """paged_decode for a batch with shared prefixes: `groups` = [(first_row, rows, shared_tokens)]
    or [([row, ...], shared_tokens)] (the finders above), or `descriptors` = the PrefixGroups made
    from them (to keep the host-to-device copy out of a step; its partition size then counts).
    Partitions inside a group's shared prefix are read once per group.  Same result as
    paged_decode(partition_size=partition_size).  The groups are trusted; PA_DEBUG_TABLES=1 checks
    them against the tables before every launch.  longest_context: the host's bound on context_lens;
    the launch is then sized for rows that long instead of for the table's width (a longer row is still
    computed exactly, its last partition runs to the row's end)."""
    _require_gpu(q, "paged_decode_shared_prefix")
    _require_gpu(k_cache, "paged_decode_shared_prefix")
    _check_cache(k_cache, v_cache, "paged_decode_shared_prefix")
    lib = _native.load()
    if q.dim() != 3:
        raise RuntimeError("paged_decode_shared_prefix: q must be [batch, heads, head_dim]")
    batch, num_q_heads, head_dim = q.shape
    num_blocks, block_size, num_kv_heads, d2 = k_cache.shape
    if d2 != head_dim:
        raise RuntimeError("paged_decode_shared_prefix: q head_dim %d != cache head_dim %d" % (head_dim, d2))
    if block_tables.dim() != 2 or block_tables.shape[0] != batch or context_lens.numel() != batch:
        raise RuntimeError("paged_decode_shared_prefix: block_tables/context_lens do not match the batch")
    if descriptors is None:
        descriptors = shared_prefix_descriptors(groups, batch, q.device, int(partition_size))
    pg = descriptors
    psize = pg.partition_size
    if psize <= 0 or psize % 16 or psize % block_size:
        raise RuntimeError("paged_decode_shared_prefix: partition_size must be a multiple of 16 and of the block size")
    if pg.batch < batch:
        raise RuntimeError("paged_decode_shared_prefix: descriptors cover %d rows, the batch has %d" % (pg.batch, batch))
    q, qs = _rows(q, "paged_decode_shared_prefix")
    tables = block_tables if block_tables.dtype == torch.int32 else block_tables.to(torch.int32)
    if tables.stride(1) != 1:
        tables = tables.contiguous()
    lens = _int32(context_lens, "paged_decode_shared_prefix")
    if out is None:
        out = torch.empty((batch, num_q_heads, head_dim), dtype=q.dtype, device=q.device)
    if batch == 0:
        return out
    kv_code = _code(k_cache.dtype, "paged_decode_shared_prefix")
    fp8 = kv_code == _native.DTYPE_FP8_E4M3
    if fp8 and (k_scale is None or v_scale is None):
        raise RuntimeError("paged_decode_shared_prefix: fp8 cache needs k_scale and v_scale")
    parts = max(1, (tables.shape[1] * block_size + psize - 1) // psize)
    if longest_context:
        # every row needs a partition of its own after the shared ones, for what it holds beyond the bound
        bound, _ = _known_lengths(tables.shape[1] * block_size, longest_context, None)
        parts = min(parts, max((bound + psize - 1) // psize, pg.max_shared_partitions + 1))
    rows_ptr = pg.group_rows.data_ptr() if pg.group_rows is not None else None
    rows_len = pg.group_rows.numel() if pg.group_rows is not None else 0
    if _debug_tables():
        counts = torch.zeros(3, dtype=torch.int32, device=q.device)
        rc = lib.pa_check_shared_prefix(tables.data_ptr(), tables.stride(0), tables.shape[1], lens.data_ptr(), batch,
                                        block_size, psize, pg.group_desc.data_ptr(), pg.num_groups, rows_ptr, rows_len,
                                        pg.row_skip.data_ptr(), counts.data_ptr(), _stream_ptr(q.device))
        _native.check(rc, "pa_check_shared_prefix")
        differ, short, stray = counts.tolist()
        if differ or short or stray:
            raise RuntimeError("paged_decode_shared_prefix: %d shared table entries differ inside their group, %d rows "
                               "too short for their group or with the wrong row_skip, %d rows outside the groups "
                               "with a row_skip or inside two groups" % (differ, short, stray))
    ws_bytes = lib.pa_workspace_bytes(batch, num_q_heads, head_dim, parts)
    if workspace is not None:
        if workspace.dtype != torch.uint8 or not workspace.is_cuda or workspace.numel() < ws_bytes:
            raise RuntimeError("paged_decode_shared_prefix: workspace must be a uint8 GPU tensor of at least %d bytes" % ws_bytes)
        ws = workspace
    else:
        ws = reserve_decode_workspace(q.device, ws_bytes)
    own = max(1, parts - pg.min_row_skip)      # every row computes what its group does not
    rc = lib.pa_decode_shared_prefix(q.data_ptr(), _code(q.dtype, "paged_decode_shared_prefix"), qs, k_cache.data_ptr(),
                                     v_cache.data_ptr(), k_scale.data_ptr() if fp8 else None,
                                     v_scale.data_ptr() if fp8 else None, kv_code, tables.data_ptr(),
                                     tables.stride(0), tables.shape[1], lens.data_ptr(), out.data_ptr(), out.stride(0),
                                     batch, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, float(scale),
                                     psize, parts, ws.data_ptr(), ws_bytes, int(waves or 0), pg.group_desc.data_ptr(),
                                     pg.num_groups, rows_ptr, rows_len, max(1, pg.max_group_rows),
                                     min(pg.max_shared_partitions, parts), pg.row_skip.data_ptr(), own,
                                     _stream_ptr(q.device))
    _native.check(rc, "pa_decode_shared_prefix")
    return out


def paged_decode(q, k_cache, v_cache, block_tables, context_lens, scale, k_scale=None,
                 v_scale=None, partition_size=None, out=None, waves=0, kv_heads_per_wave=None,
                 q_heads_per_wave=0, workspace=None, longest_context=None, mean_context=None):
    """Decode attention of q [batch, heads, head_dim] against the paged cache.

    partition_size None: single pass, or an automatic split when the batch alone cannot fill
    the GPU (same result up to fp32 rounding).  partition_size > 0: the partitioned algorithm
    of src/inference/attention.py:434-626 with that size.  Never synchronises with the host.
    waves / kv_heads_per_wave / q_heads_per_wave shape the launch (0 or None: the launch policy's
    choice); they never change the result.  workspace: a uint8 tensor for the partition partials
    instead of the device's shared one.  longest_context / mean_context: what the host knows about
    context_lens (upper bound, mean) - the launch is then sized for the rows instead of for the
    table's width (choose_partition); wrong values cost time, never correctness.
    """
    _require_gpu(q, "paged_decode")
    _require_gpu(k_cache, "paged_decode")
    _check_cache(k_cache, v_cache, "paged_decode")
    lib = _native.load()
    if q.dim() != 3:
        raise RuntimeError("paged_decode: q must be [batch, heads, head_dim]")
    batch, num_q_heads, head_dim = q.shape
    num_blocks, block_size, num_kv_heads, d2 = k_cache.shape
    if d2 != head_dim:
        raise RuntimeError("paged_decode: q head_dim %d != cache head_dim %d" % (head_dim, d2))
    if block_tables.dim() != 2 or block_tables.shape[0] != batch or context_lens.numel() != batch:
        raise RuntimeError("paged_decode: block_tables/context_lens do not match the batch")
    q, qs = _rows(q, "paged_decode")
    tables = block_tables if block_tables.dtype == torch.int32 else block_tables.to(torch.int32)
    if tables.stride(1) != 1:
        tables = tables.contiguous()
    lens = _int32(context_lens, "paged_decode")
    if out is None:
        out = torch.empty((batch, num_q_heads, head_dim), dtype=q.dtype, device=q.device)
    if batch == 0:
        return out
    kv_code = _code(k_cache.dtype, "paged_decode")
    fp8 = kv_code == _native.DTYPE_FP8_E4M3
    if fp8 and (k_scale is None or v_scale is None):
        raise RuntimeError("paged_decode: fp8 cache needs k_scale and v_scale")
    if _debug_tables():
        bad, short = check_block_tables(tables, lens, block_size, num_blocks)
        if bad or short:
            raise RuntimeError("paged_decode: %d block-table entries outside the pool of %d blocks, %d rows whose "
                               "context_len needs more than the table's %d columns"
                               % (bad, num_blocks, short, tables.shape[1]))
    max_context = tables.shape[1] * block_size
    hpw = kv_heads_per_wave
    if partition_size is None:
        # what the policy says for this shape, replayed from a graph and (small launches that the
        # graph would split only) issued call by call; remembered per shape: the policy's own cache
        # still costs the host 1 us a call, which shows in the launches that last 10 us
        key = (batch, num_q_heads, num_kv_heads, max_context, head_dim, k_cache.element_size(), q.device.index,
               longest_context, mean_context)
        shapes = _LAUNCH_SHAPES.get(key)
        if shapes is None:
            args = (batch, num_q_heads, num_kv_heads, max_context, head_dim, k_cache.element_size(),
                    _compute_units(q.device), longest_context, mean_context)
            replayed = choose_launch(*args)
            small = replayed[1] > 1 and batch * max_context <= _EAGER_CHECK_TOKENS
            shapes = (replayed, choose_launch(*args, eager=True) if small else None)
            if len(_LAUNCH_SHAPES) >= 4096:
                _LAUNCH_SHAPES.clear()
            _LAUNCH_SHAPES[key] = shapes
        psize, parts, auto_hpw = shapes[0]
        # outside a graph capture the second launch of a split costs the host more than the split saves
        # on the device (a warm-up inside sizing_graph_workspace() stands for the capture that follows:
        # the same split)
        if shapes[1] is not None and not _sizing_for_graphs and not _is_capturing():
            psize, parts, auto_hpw = shapes[1]
        if hpw is None:
            hpw = auto_hpw
    else:
        psize = int(partition_size)
        bound, _ = _known_lengths(max_context, longest_context, None)
        parts = max(1, (bound + psize - 1) // psize)
    ws_ptr, ws_bytes = None, 0
    if parts > 1:
        ws_bytes = lib.pa_workspace_bytes(batch, num_q_heads, head_dim, parts)
        if workspace is not None:
            if workspace.dtype != torch.uint8 or not workspace.is_cuda or workspace.numel() < ws_bytes:
                raise RuntimeError("paged_decode: workspace must be a uint8 GPU tensor of at least %d bytes" % ws_bytes)
            ws = workspace
        else:
            ws = reserve_decode_workspace(q.device, ws_bytes)
        ws_ptr = ws.data_ptr()
    rc = lib.pa_decode(q.data_ptr(), _code(q.dtype, "paged_decode"), qs, k_cache.data_ptr(),
                       v_cache.data_ptr(), k_scale.data_ptr() if fp8 else None,
                       v_scale.data_ptr() if fp8 else None, kv_code, tables.data_ptr(),
                       tables.stride(0), tables.shape[1], lens.data_ptr(), out.data_ptr(), out.stride(0),
                       batch, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, float(scale),
                       psize, parts, ws_ptr, ws_bytes, int(waves or 0), int(hpw or 0),
                       int(q_heads_per_wave or 0), _stream_ptr(q.device))
    _native.check(rc, "pa_decode")
    return out


def paged_prefill(q, k_src, v_src, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, scale,
                  block_tables=None, k_scale=None, v_scale=None, out=None, waves=0):
    """Causal varlen prefill attention on the MFMA kernel.

    q [total_new_tokens, heads, head_dim]; cu_seqlens_q / cu_seqlens_k int32 [num_seqs + 1]
    (new tokens, and cached + new tokens, per sequence).  With block_tables, k_src / v_src are
    the paged caches [num_blocks, block_size, kv_heads, head_dim] and row i of a chunk sees the
    cached prefix plus the chunk up to itself; without, they are the dense new-token tensors
    [total_k_tokens, kv_heads, head_dim] (src/inference/attention.py:243-257).
    waves: 0 = the launch's own choice of waves per workgroup, or 4 / 8; never changes the result.
    """
    _require_gpu(q, "paged_prefill")
    _require_gpu(k_src, "paged_prefill")
    lib = _native.load()
    if q.dim() != 3:
        raise RuntimeError("paged_prefill: q must be [tokens, heads, head_dim]")
    total_q, num_q_heads, head_dim = q.shape
    q, qs = _rows(q, "paged_prefill")
    if out is None:
        out = torch.empty((total_q, num_q_heads, head_dim), dtype=q.dtype, device=q.device)
    if total_q == 0:
        return out
    cu_q = _int32(cu_seqlens_q, "paged_prefill")
    cu_k = _int32(cu_seqlens_k, "paged_prefill")
    num_seqs = cu_q.numel() - 1
    if cu_k.numel() != num_seqs + 1:
        raise RuntimeError("paged_prefill: cu_seqlens_q and cu_seqlens_k differ in length")
    kv_code = _code(k_src.dtype, "paged_prefill")
    fp8 = kv_code == _native.DTYPE_FP8_E4M3
    if block_tables is not None:
        _check_cache(k_src, v_src, "paged_prefill")
        num_blocks, block_size, num_kv_heads, d2 = k_src.shape
        tables = block_tables if block_tables.dtype == torch.int32 else block_tables.to(torch.int32)
        if tables.stride(1) != 1:
            tables = tables.contiguous()
        bt_ptr, bt_stride = tables.data_ptr(), tables.stride(0)
        if fp8 and (k_scale is None or v_scale is None):
            raise RuntimeError("paged_prefill: fp8 cache needs k_scale and v_scale")
        kp, vp = k_src, v_src
    else:
        if k_src.dim() != 3 or v_src.shape != k_src.shape or k_src.dtype != v_src.dtype:
            raise RuntimeError("paged_prefill: dense k/v must both be [tokens, kv_heads, head_dim]")
        kp, kstride = _rows(k_src, "paged_prefill")
        vp, vstride = _rows(v_src, "paged_prefill")
        if vstride != kstride:
            vp = vp.contiguous()
            kp = kp.contiguous()
            kstride = kp.shape[1] * kp.shape[2]
        num_kv_heads, d2 = kp.shape[1], kp.shape[2]
        num_blocks, block_size = 1, 1
        bt_ptr, bt_stride = None, kstride
    if d2 != head_dim:
        raise RuntimeError("paged_prefill: q head_dim %d != k/v head_dim %d" % (head_dim, d2))
    rc = lib.pa_prefill(q.data_ptr(), _code(q.dtype, "paged_prefill"), qs, kp.data_ptr(),
                        vp.data_ptr(), k_scale.data_ptr() if fp8 else None,
                        v_scale.data_ptr() if fp8 else None, kv_code, bt_ptr, bt_stride,
                        cu_q.data_ptr(), cu_k.data_ptr(), out.data_ptr(), out.stride(0), num_seqs,
                        int(max_seqlen_q), num_q_heads, num_kv_heads, head_dim, block_size,
                        num_blocks, float(scale), int(waves or 0), _stream_ptr(q.device))
    _native.check(rc, "pa_prefill")
    return out


# ==================== modules ====================

class PagedAttention(nn.Module):
    """Attention layer of the inference engine: writes the new K/V into the paged cache, then
    runs varlen prefill or single-token decode according to the global context.

    k_cache / v_cache / k_scale / v_scale / cache_dtype are bound by the model runner
    (src/inference/model_runner.py:102-116).
    """

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int,
                 cache_dtype: str = "fp16"):
        super().__init__()
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.scale = head_dim ** -0.5
        self.cache_dtype = cache_dtype
        self.k_cache: Optional[torch.Tensor] = None
        self.v_cache: Optional[torch.Tensor] = None
        self.k_scale: Optional[torch.Tensor] = None
        self.v_scale: Optional[torch.Tensor] = None

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        """q [tokens, heads, dim], k/v [tokens, kv_heads, dim] -> [tokens, heads, dim]."""
        ctx = get_context()
        # the write precedes the read: context_lens already counts the new token
        if self.k_cache is not None and ctx.slot_mapping is not None:
            store_kv_cache(k, v, self.k_cache, self.v_cache, ctx.slot_mapping,
                           k_scale=self.k_scale, v_scale=self.v_scale,
                           cache_dtype=self.cache_dtype)
        if ctx.is_prefill:
            return self._prefill_attention(q, k, v, ctx)
        return self._decode_attention(q, ctx)

    def forward_fused(self, q, k, v, q_norm_weight, k_norm_weight, eps, inv_freq, positions):
        """forward() for projections that still need their per-head RMSNorm and rotary embedding:
        norm, rotation and the cache write run as one kernel, then attention as in forward()."""
        ctx = get_context()
        write = self.k_cache is not None and ctx.slot_mapping is not None
        dense_k = ctx.is_prefill and not (ctx.block_tables is not None and self.k_cache is not None)
        q, k_rot = qk_norm_rope_store(
            q, k, v, q_norm_weight, k_norm_weight, eps, inv_freq, positions,
            k_cache=self.k_cache if write else None, v_cache=self.v_cache if write else None,
            slot_mapping=ctx.slot_mapping if write else None, k_scale=self.k_scale, v_scale=self.v_scale,
            cache_dtype=self.cache_dtype, return_k=dense_k)
        if ctx.is_prefill:
            return self._prefill_attention(q, k_rot, v, ctx)
        return self._decode_attention(q, ctx)

    def _scales(self):
        if self.cache_dtype == "fp8" and self.k_scale is not None:
            return self.k_scale, self.v_scale
        return None, None

    def _prefill_attention(self, q, k, v, ctx):
        if ctx.block_tables is not None and self.k_cache is not None:
            ks, vs = self._scales()
            return paged_prefill(q, self.k_cache, self.v_cache, ctx.cu_seqlens_q, ctx.cu_seqlens_k,
                                 ctx.max_seqlen_q, self.scale, block_tables=ctx.block_tables,
                                 k_scale=ks, v_scale=vs)
        return paged_prefill(q, k, v, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.max_seqlen_q,
                             self.scale)

    def _decode_attention(self, q, ctx):
        if self.k_cache is None or ctx.block_tables is None or ctx.context_lens is None:
            return q  # nothing bound: same last-resort behaviour as attention.py:329-330
        ks, vs = self._scales()
        shared = self._shared_prefix_decode(q, ctx, ks, vs)
        if shared is not None:
            return shared
        return paged_decode(q, self.k_cache, self.v_cache, ctx.block_tables, ctx.context_lens,
                            self.scale, k_scale=ks, v_scale=vs,
                            longest_context=getattr(ctx, "longest_context_len", 0) or None,
                            mean_context=getattr(ctx, "mean_context_len", 0) or None)

    def _shared_prefix_decode(self, q, ctx, ks, vs):
        """Rows that share prefixes (ctx.prefix_groups, set by the runner when it found any): the shared
        partitions are read once per group.  None when the step has no groups."""
        pg = getattr(ctx, "prefix_groups", None)
        if pg is None or q.shape[0] > pg.batch or 16 // max(1, self.num_heads // self.num_kv_heads) < pg.max_group_rows:
            return None
        return paged_decode_shared_prefix(q, self.k_cache, self.v_cache, ctx.block_tables, ctx.context_lens,
                                          self.scale, None, k_scale=ks, v_scale=vs, descriptors=pg,
                                          longest_context=getattr(ctx, "longest_context_len", 0) or None)


class PartitionedPagedAttention(PagedAttention):
    """Decode attention split into partitions of `partition_size` tokens with an exact
    log-sum-exp merge (src/inference/attention.py:387-626).

    The reference picks the path after a host read of max(context_lens); here the launch is
    sized from the block-table width instead, so no host synchronisation happens: sequences
    shorter than one partition simply own a single partition, which merges to itself.

    The merge is exact, so the split is the launch policy's to choose (choose_partition): none at
    256 sequences, where 512-token partitions only add partial results to write and merge; 64 to
    128 tokens for one or two sequences, where a round of short workgroups beats a few long ones.
    `adaptive = False` keeps every launch at exactly partition_size, the reference's split.
    """

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int,
                 cache_dtype: str = "fp16", partition_size: int = 512):
        super().__init__(num_heads, num_kv_heads, head_dim, cache_dtype)
        self.partition_size = partition_size
        self.adaptive = True

    def _decode_attention(self, q, ctx):
        if ctx.context_lens is None:
            return super()._decode_attention(q, ctx)
        return self._partitioned_decode(q, ctx)

    def _partitioned_decode(self, q, ctx):
        if self.k_cache is None or ctx.block_tables is None or ctx.context_lens is None:
            return q
        ks, vs = self._scales()
        shared = self._shared_prefix_decode(q, ctx, ks, vs)
        if shared is not None:
            return shared
        longest = getattr(ctx, "longest_context_len", 0) or None
        mean = getattr(ctx, "mean_context_len", 0) or None
        psize = None if self.adaptive else self.partition_size      # None: the launch policy's split
        return paged_decode(q, self.k_cache, self.v_cache, ctx.block_tables, ctx.context_lens,
                            self.scale, k_scale=ks, v_scale=vs, partition_size=psize,
                            longest_context=longest, mean_context=mean)
