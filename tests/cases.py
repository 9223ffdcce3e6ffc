"""Seeded synthetic paged-attention cases shared by the tests, the smoke check and the bench.

Everything is generated on the CPU from a torch.Generator seed so that the oracle and the GPU
path see identical bits; the pool is filled through the oracle's store (fp16 copy or fp8
quantisation), unused pool blocks and the unused tail of each last block are poisoned
(NaN for 16-bit caches, byte 0x7F = NaN for fp8, NaN scales) so that any read outside a
sequence's context shows up as NaN in the output.
"""
import math

import torch

from oracle import paged_attention_oracle as oracle

FP8 = torch.float8_e4m3fn


def poison_(t):
    if t.dtype == FP8:
        t.view(torch.uint8).fill_(0x7F)
    else:
        t.fill_(float("nan"))
    return t


def build_tables(gen, context_lens, num_blocks, block_size, pad=-1, extra_cols=0, shared_prefix=None):
    """Random-permutation block tables.  shared_prefix = (group_size, prefix_blocks): sequences
    of one group map their first prefix_blocks table entries to the same physical blocks."""
    batch = len(context_lens)
    need = [(int(c) + block_size - 1) // block_size for c in context_lens]
    width = max(max(need), 1) + extra_cols
    perm = torch.randperm(num_blocks, generator=gen).tolist()
    tables = torch.full((batch, width), pad, dtype=torch.int32)
    cursor = 0
    owners = []          # per sequence: list of (logical block, physical block) it writes itself
    for b in range(batch):
        own = []
        for j in range(need[b]):
            if shared_prefix and j < shared_prefix[1] and b % shared_prefix[0] != 0:
                tables[b, j] = tables[b - b % shared_prefix[0], j]
                continue
            assert cursor < num_blocks, "pool too small for the case"
            tables[b, j] = perm[cursor]
            own.append((j, perm[cursor]))
            cursor += 1
        owners.append(own)
    return tables, owners, perm[cursor:]


def make_case(seed, context_lens, num_blocks, block_size=16, num_heads=16, num_kv_heads=8,
              head_dim=128, cache="fp16", q_dtype=torch.float16, pad=-1, extra_cols=0,
              shared_prefix=None, per_tensor_scale=False, poison=True):
    """Returns a dict of CPU tensors: q, k_cache, v_cache, k_scale, v_scale, block_tables,
    context_lens, scale, cache_dtype (+ keys/values per sequence for brute-force checks)."""
    gen = torch.Generator().manual_seed(seed)
    batch = len(context_lens)
    kv_dtype = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp8": FP8}[cache]
    src_dtype = torch.float16 if cache == "fp8" else kv_dtype
    shape = (num_blocks, block_size, num_kv_heads, head_dim)
    k_cache = torch.zeros(shape, dtype=kv_dtype)
    v_cache = torch.zeros(shape, dtype=kv_dtype)
    k_scale = v_scale = None
    if poison:
        poison_(k_cache)
        poison_(v_cache)
    if cache == "fp8":
        k_scale = torch.full((num_blocks, block_size), float("nan") if poison else 1.0)
        v_scale = torch.full((num_blocks, block_size), float("nan") if poison else 1.0)
    tables, owners, _free = build_tables(gen, context_lens, num_blocks, block_size, pad,
                                         extra_cols, shared_prefix)
    for b in range(batch):
        n = int(context_lens[b])
        if n <= 0:
            continue
        # tokens this sequence writes itself (everything except an aliased prefix)
        first_own = 0
        if shared_prefix and b % shared_prefix[0] != 0:
            first_own = min(shared_prefix[1] * block_size, n)
        cnt = n - first_own
        if cnt <= 0:
            continue
        k = torch.randn(cnt, num_kv_heads, head_dim, generator=gen).to(src_dtype)
        v = torch.randn(cnt, num_kv_heads, head_dim, generator=gen).to(src_dtype)
        pos = torch.arange(first_own, n)
        slots = (tables[b, pos // block_size].long() * block_size + pos % block_size).to(torch.int32)
        if cache == "fp8" and per_tensor_scale:
            # one amax/448-style scale for the whole tensor, replicated into every token slot
            s_k = 448.0 / k.float().abs().max().clamp(min=1e-5)
            s_v = 448.0 / v.float().abs().max().clamp(min=1e-5)
            k_cache.view(-1, num_kv_heads, head_dim)[slots.long()] = (k.float() * s_k).to(FP8)
            v_cache.view(-1, num_kv_heads, head_dim)[slots.long()] = (v.float() * s_v).to(FP8)
            k_scale.view(-1)[slots.long()] = s_k
            v_scale.view(-1)[slots.long()] = s_v
        else:
            oracle.store_kv_cache(k, v, k_cache, v_cache, slots, k_scale, v_scale,
                                  "fp8" if cache == "fp8" else "fp16")
    q = torch.randn(batch, num_heads, head_dim, generator=gen).to(q_dtype)
    return {
        "q": q, "k_cache": k_cache, "v_cache": v_cache, "k_scale": k_scale, "v_scale": v_scale,
        "block_tables": tables, "context_lens": torch.tensor([int(c) for c in context_lens], dtype=torch.int32),
        "scale": 1.0 / math.sqrt(head_dim), "cache_dtype": "fp8" if cache == "fp8" else "fp16",
        "block_size": block_size, "num_blocks": num_blocks,
    }


def to_device(case, device):
    out = {}
    for k, v in case.items():
        out[k] = v.to(device) if isinstance(v, torch.Tensor) else v
    return out


def uniform_lens(seed, batch, lo, hi):
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (batch,), generator=gen).tolist()


# The five benchmark configurations (decode side), by name.
def config1(seed=1001):
    """bs 8, ctx U[128,512], pool of 512 blocks, fp16 KV."""
    return make_case(seed, uniform_lens(seed, 8, 128, 512), 512)


def config2(seed=1002, cache="fp8", batch=64, ctx=4096, spare=64, **kw):
    """bs 64, ctx 4096, fp8 KV quantised by the store (headline shape)."""
    blocks = batch * ((ctx + 15) // 16) + spare
    return make_case(seed, [ctx] * batch, blocks, cache=cache, **kw)


def config3(seed=1003, batch=4, lo=16384, hi=32768):
    """bs 4, ctx U[16384,32768], fp16 KV, for the partitioned path."""
    lens = uniform_lens(seed, batch, lo, hi)
    blocks = sum((c + 15) // 16 for c in lens) + 64
    return make_case(seed, lens, blocks)


def config4(seed=1004, prompts=32, samples=8, prefix=1024, lo=64, hi=512, cache="fp16"):
    """32 prompts x 8 samples sharing a 1024-token prefix (aliased physical blocks)."""
    suffix = uniform_lens(seed, prompts * samples, lo, hi)
    lens = [prefix + s for s in suffix]
    own = sum((l + 15) // 16 - (prefix // 16 if i % samples else 0) for i, l in enumerate(lens))
    return make_case(seed, lens, own + 64, shared_prefix=(samples, prefix // 16), cache=cache)
