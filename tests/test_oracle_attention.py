"""Pins the oracle's attention functions by closed forms, invariants and brute force
(the reference holds no golden vectors for this path)."""
import math

import pytest
import torch

import cases
from oracle import paged_attention_oracle as oracle


def small_case(seed=3, cache="fp16", lens=(1, 5, 16, 17, 40), nb=16, **kw):
    return cases.make_case(seed, list(lens), num_blocks=nb, block_size=8, num_heads=4,
                           num_kv_heads=2, head_dim=16, cache=cache, q_dtype=torch.float32, **kw)


def run_decode(c):
    return oracle.decode(c["q"], c["k_cache"], c["v_cache"], c["block_tables"], c["context_lens"],
                         c["scale"], c["k_scale"], c["v_scale"], c["cache_dtype"])


def test_fp16_store_is_a_scatter_copy():
    g = torch.Generator().manual_seed(1)
    k = torch.randn(6, 2, 16, generator=g).half()
    v = torch.randn(6, 2, 16, generator=g).half()
    kc = torch.full((4, 8, 2, 16), 7.0, dtype=torch.float16)
    vc = torch.full((4, 8, 2, 16), 7.0, dtype=torch.float16)
    slots = torch.tensor([31, -1, 0, 9, -1, 16], dtype=torch.int32)
    oracle.store_kv_cache(k, v, kc, vc, slots)
    flat_k, flat_v = kc.view(32, 2, 16), vc.view(32, 2, 16)
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            assert torch.equal(flat_k[s], k[t]) and torch.equal(flat_v[s], v[t])
    untouched = [s for s in range(32) if s not in (31, 0, 9, 16)]
    assert bool((flat_k[untouched] == 7).all()) and bool((flat_v[untouched] == 7).all())


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_decode_matches_fp64_brute_force(cache):
    c = small_case(cache=cache)
    got = run_decode(c).double()
    want = oracle.decode_f64(c["q"], c["k_cache"], c["v_cache"], c["block_tables"],
                             c["context_lens"], c["scale"], c["k_scale"], c["v_scale"])
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-5)


def test_decode_ctx1_returns_v0_of_the_mapped_kv_head():
    c = small_case(lens=(1, 1, 1))
    out = run_decode(c)
    for b in range(3):
        blk = int(c["block_tables"][b, 0])
        v0 = c["v_cache"][blk, 0].float()           # [Hkv, D]
        for h in range(4):
            assert torch.allclose(out[b, h], v0[h // 2], atol=1e-6)


def test_decode_invariant_under_physical_block_permutation():
    c = small_case()
    base = run_decode(c)
    perm = torch.randperm(16, generator=torch.Generator().manual_seed(5))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(16)
    c2 = dict(c)
    c2["k_cache"] = c["k_cache"][perm]
    c2["v_cache"] = c["v_cache"][perm]
    t = c["block_tables"].clone()
    valid = t >= 0
    t[valid] = inv[t[valid].long()].to(torch.int32)
    c2["block_tables"] = t
    assert torch.equal(run_decode(c2), base)


def test_decode_ignores_table_tail_and_unused_blocks():
    c = small_case(extra_cols=3)
    base = run_decode(c)
    assert not torch.isnan(base).any()          # pool poison never reached
    c2 = dict(c)
    t = c["block_tables"].clone()
    t[t < 0] = 9                                 # stale / zero padding instead of -1
    c2["block_tables"] = t
    assert torch.equal(run_decode(c2), base)


def test_decode_zero_context_row_is_zero():
    c = small_case(lens=(0, 9))
    out = run_decode(c)
    assert float(out[0].abs().max()) == 0.0 and float(out[1].abs().max()) > 0.0


def test_partition_lse_and_single_partition_identity():
    c = small_case(lens=(40,))
    q = c["q"][0:1]
    out, lse = oracle.partition_attention(q, c["k_cache"], c["v_cache"], c["block_tables"][0], 0, 40,
                                          8, c["scale"])
    full = run_decode(c)
    assert torch.allclose(out, full, rtol=1e-5, atol=1e-6)
    assert torch.allclose(oracle.merge_partitions([out], [lse]), out, rtol=1e-6, atol=1e-7)
    # lse == log(sum(exp(scores))) from first principles
    flat = oracle._flat_indices(c["block_tables"][0], 0, 40, 8)
    K = c["k_cache"].view(-1, 2, 16)[flat].double()
    for h in range(4):
        s = (K[:, h // 2] @ q[0, h].double()) * c["scale"]
        assert math.isclose(float(lse[0, h]), float(torch.log(torch.exp(s).sum())), rel_tol=1e-5)


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
@pytest.mark.parametrize("psize", [8, 16, 24])
def test_partitioned_equals_single_pass(cache, psize):
    c = small_case(cache=cache, lens=(3, 8, 9, 40, 64), nb=24)
    single = run_decode(c)
    part = oracle.decode_partitioned(c["q"], c["k_cache"], c["v_cache"], c["block_tables"],
                                     c["context_lens"], c["scale"], psize, c["k_scale"],
                                     c["v_scale"], c["cache_dtype"])
    assert torch.allclose(part, single, rtol=1e-5, atol=1e-6)


def test_prefill_paged_rows_equal_decode_at_growing_context():
    # row i of the chunk == decode with context_len = cached + i + 1 (bottom-right causal)
    c = small_case(lens=(29,))
    cached, new = 17, 12
    g = torch.Generator().manual_seed(11)
    q = torch.randn(new, 4, 16, generator=g)
    cu_q = torch.tensor([0, new], dtype=torch.int32)
    cu_k = torch.tensor([0, cached + new], dtype=torch.int32)
    out = oracle.prefill_paged(q, c["k_cache"], c["v_cache"], c["block_tables"], cu_q, cu_k, c["scale"])
    for i in range(new):
        row = oracle.decode(q[i:i + 1], c["k_cache"], c["v_cache"], c["block_tables"],
                            torch.tensor([cached + i + 1], dtype=torch.int32), c["scale"])
        assert torch.allclose(out[i], row[0], rtol=1e-5, atol=1e-6)


def test_prefill_paged_without_prefix_equals_plain_causal_sdpa():
    lens = (9, 16)
    c = small_case(lens=lens)
    g = torch.Generator().manual_seed(12)
    total = sum(lens)
    q = torch.randn(total, 4, 16, generator=g)
    cu = torch.tensor([0, 9, 25], dtype=torch.int32)
    # dense K/V of the same tokens, gathered back out of the cache
    ks, vs = [], []
    for b, n in enumerate(lens):
        flat = oracle._flat_indices(c["block_tables"][b], 0, n, 8)
        ks.append(c["k_cache"].view(-1, 2, 16)[flat].float())
        vs.append(c["v_cache"].view(-1, 2, 16)[flat].float())
    dense = oracle.prefill_no_prefix(q, torch.cat(ks), torch.cat(vs), cu, cu, c["scale"])
    paged = oracle.prefill_paged(q, c["k_cache"], c["v_cache"], c["block_tables"], cu, cu, c["scale"])
    assert torch.allclose(paged, dense, rtol=1e-5, atol=1e-6)


def test_shared_prefix_tables_alias_and_stores_stay_private():
    lens = [32 + s for s in (3, 9, 1, 16)]
    c = cases.make_case(21, lens, num_blocks=24, block_size=8, num_heads=4, num_kv_heads=2,
                        head_dim=16, q_dtype=torch.float32, shared_prefix=(4, 4))
    t = c["block_tables"]
    for b in range(1, 4):
        assert torch.equal(t[b, :4], t[0, :4])
        assert len(set(t[b, 4:][t[b, 4:] >= 0].tolist()) & set(t[0].tolist())) == 0
    out = run_decode(c)
    want = oracle.decode_f64(c["q"], c["k_cache"], c["v_cache"], t, c["context_lens"], c["scale"])
    assert torch.allclose(out.double(), want, rtol=1e-5, atol=1e-5)
