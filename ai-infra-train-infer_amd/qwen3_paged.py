"""A Qwen3-shaped decoder whose attention layers are PagedAttention modules.

The reference ships no model that owns a PagedAttention (its kv_cache mode drives a
HuggingFace model and gathers KV in Python, src/inference/model_runner.py:340-433), so this is
the module a model runner binds caches to (model_runner.py:102-116) and calls as
`model(input_ids, positions=positions)` (model_runner.py:162).  Block structure follows the
reference's Qwen3 definition (src/distributed/tensor_parallel.py:307-543): RMSNorm -> q/k/v
projections -> per-head q/k RMSNorm -> RoPE (half rotation, theta 1e6) -> attention -> o_proj,
then RMSNorm -> SwiGLU MLP.  GEMMs are torch-ROCm library calls.  Between them a block runs
five HIP kernels: residual add + RMSNorm, per-head q/k norm + rotation + KV write (`fused_qk`),
attention, residual add + RMSNorm again, and silu(gate) * up (`fused_elementwise`); both flags are
on by default, off = the same steps as separate torch ops.  The residual add of a block's MLP
output is carried into the next block's first norm (and the last one into the final norm), so
no add is a launch of its own.  Nothing in forward() synchronises with the host, so a decode
step can be captured in a HIP graph.
"""
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F

from .attention import PagedAttention, PartitionedPagedAttention, add_rms_norm, silu_mul
from .context import get_context


@dataclass
class Qwen3PagedConfig:
    """Defaults are the Qwen3-0.6B shape."""
    vocab_size: int = 151936
    hidden_size: int = 1024
    intermediate_size: int = 3072
    num_layers: int = 28
    num_heads: int = 16
    num_kv_heads: int = 8
    head_dim: int = 128
    rope_theta: float = 1000000.0
    rms_norm_eps: float = 1e-6
    cache_dtype: str = "fp16"
    partition_size: int = 0        # > 0: use PartitionedPagedAttention with this size
    fused_qk: bool = True          # q/k norm + RoPE + cache write as one kernel
    fused_elementwise: bool = True # residual add + RMSNorm, and silu * up, as one kernel each


class RMSNorm(nn.Module):
    def __init__(self, dim, eps):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)
        return (xf * self.weight.float()).to(x.dtype)


def apply_rope(x, cos, sin):
    """x [T, H, D]; cos/sin [T, 1, D] (frequencies repeated over both halves)."""
    half = x.shape[-1] // 2
    rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    return (x.float() * cos + rot.float() * sin).to(x.dtype)


class Qwen3PagedLayer(nn.Module):
    def __init__(self, cfg: Qwen3PagedConfig):
        super().__init__()
        self.cfg = cfg
        q_dim, kv_dim = cfg.num_heads * cfg.head_dim, cfg.num_kv_heads * cfg.head_dim
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)
        self.qkv_proj = nn.Linear(cfg.hidden_size, q_dim + 2 * kv_dim, bias=False)
        self.q_norm = RMSNorm(cfg.head_dim, cfg.rms_norm_eps)
        self.k_norm = RMSNorm(cfg.head_dim, cfg.rms_norm_eps)
        if cfg.partition_size > 0:
            self.attn = PartitionedPagedAttention(cfg.num_heads, cfg.num_kv_heads, cfg.head_dim,
                                                  cfg.cache_dtype, cfg.partition_size)
        else:
            self.attn = PagedAttention(cfg.num_heads, cfg.num_kv_heads, cfg.head_dim, cfg.cache_dtype)
        self.o_proj = nn.Linear(q_dim, cfg.hidden_size, bias=False)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)
        self.gate_up_proj = nn.Linear(cfg.hidden_size, 2 * cfg.intermediate_size, bias=False)
        self.down_proj = nn.Linear(cfg.intermediate_size, cfg.hidden_size, bias=False)

    def forward(self, x, cos, sin, positions=None, inv_freq=None, delta=None):
        """x: residual stream [T, hidden]; delta: the previous block's MLP output, not yet added
        (fused_elementwise only).  Returns (x, delta) for the next block."""
        cfg = self.cfg
        t = x.shape[0]
        q_dim, kv_dim = cfg.num_heads * cfg.head_dim, cfg.num_kv_heads * cfg.head_dim
        fused_ew = cfg.fused_elementwise and x.is_cuda
        if fused_ew:
            x, normed = add_rms_norm(x, self.input_layernorm.weight, cfg.rms_norm_eps, delta)
        else:
            if delta is not None:
                x = x + delta
            normed = self.input_layernorm(x)
        qkv = self.qkv_proj(normed)
        q = qkv[:, :q_dim].view(t, cfg.num_heads, cfg.head_dim)
        k = qkv[:, q_dim:q_dim + kv_dim].view(t, cfg.num_kv_heads, cfg.head_dim)
        v = qkv[:, q_dim + kv_dim:].view(t, cfg.num_kv_heads, cfg.head_dim)
        if cfg.fused_qk and positions is not None and x.is_cuda:
            a = self.attn.forward_fused(q, k, v, self.q_norm.weight, self.k_norm.weight,
                                        cfg.rms_norm_eps, inv_freq, positions)
        else:
            q = apply_rope(self.q_norm(q), cos, sin)
            k = apply_rope(self.k_norm(k), cos, sin)
            a = self.attn(q, k, v)                  # writes k, v into the paged cache, then attends
        o = self.o_proj(a.reshape(t, q_dim))
        if fused_ew:
            x, normed = add_rms_norm(x, self.post_attention_layernorm.weight, cfg.rms_norm_eps, o)
            return x, self.down_proj(silu_mul(self.gate_up_proj(normed)))
        x = x + o
        gu = self.gate_up_proj(self.post_attention_layernorm(x))
        gate, up = gu[:, :cfg.intermediate_size], gu[:, cfg.intermediate_size:]
        return x + self.down_proj(F.silu(gate) * up), None


class Qwen3PagedModel(nn.Module):
    """model(input_ids [T], positions=[T]) -> logits.  Decode: [T, vocab].  Prefill: one row per
    sequence (its last new token), found from the context's cu_seqlens_q."""

    def __init__(self, cfg: Qwen3PagedConfig):
        super().__init__()
        self.cfg = cfg
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = nn.ModuleList(Qwen3PagedLayer(cfg) for _ in range(cfg.num_layers))
        self.norm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)
        self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False)
        inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, dtype=torch.float32)
                                             / cfg.head_dim))
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    def rope_tables(self, positions):
        freqs = positions.float()[:, None] * self.inv_freq[None, :]
        emb = torch.cat([freqs, freqs], dim=-1)
        return emb.cos()[:, None, :], emb.sin()[:, None, :]

    def forward(self, input_ids, positions=None):
        if positions is None:
            positions = torch.arange(input_ids.shape[0], device=input_ids.device)
        fused = self.cfg.fused_qk and input_ids.is_cuda
        cos, sin = (None, None) if fused else self.rope_tables(positions)
        x = self.embed_tokens(input_ids)
        # a model cast with .half() carries its frequency table in 16 bits; both paths use those values
        inv_freq = self.inv_freq.float()
        delta = None
        for layer in self.layers:
            x, delta = layer(x, cos, sin, positions, inv_freq, delta)
        ctx = get_context()
        if ctx.is_prefill and ctx.cu_seqlens_q is not None:
            last = (ctx.cu_seqlens_q[1:] - 1).long()
            x = x[last]
            delta = delta[last] if delta is not None else None
        if self.cfg.fused_elementwise and x.is_cuda:
            x = add_rms_norm(x, self.norm.weight, self.cfg.rms_norm_eps, delta)[1]
        else:
            x = self.norm(x if delta is None else x + delta)
        return self.lm_head(x)
