"""Chunked-prefill paged attention (MFMA kernel) on the GPU against the oracle.

fp16 / fp32 outputs use the tolerances stated for the path (rtol 1e-3 / atol 2e-3 for 16-bit caches,
1e-2 / 1e-2 for fp8).  bf16 outputs are compared with the oracle's unrounded fp32 result and
are allowed one extra bf16 rounding (2^-8 relative) on top, since an 8-bit mantissa cannot
resolve 1e-3.
"""
import math

import pytest
import torch

import cases
from oracle import paged_attention_oracle as oracle

pytestmark = pytest.mark.gpu


def make_prefill(seed, cached, new, num_blocks, q_dtype=torch.float16, **kw):
    """Pool filled with cached+new tokens per sequence, plus the chunk's queries."""
    lens = [c + n for c, n in zip(cached, new)]
    c = cases.make_case(seed, lens, num_blocks, q_dtype=q_dtype, **kw)
    g = torch.Generator().manual_seed(seed + 5000)
    hq, d = c["q"].shape[1], c["q"].shape[2]
    c["q"] = torch.randn(sum(new), hq, d, generator=g).to(q_dtype)
    cu_q, cu_k = [0], [0]
    for n_, l_ in zip(new, lens):
        cu_q.append(cu_q[-1] + n_)
        cu_k.append(cu_k[-1] + l_)
    c["cu_q"] = torch.tensor(cu_q, dtype=torch.int32)
    c["cu_k"] = torch.tensor(cu_k, dtype=torch.int32)
    c["max_q"] = max(new)
    return c


def oracle_prefill(c, upcast=False):
    q = c["q"].float() if upcast else c["q"]
    return oracle.prefill_paged(q, c["k_cache"], c["v_cache"], c["block_tables"], c["cu_q"], c["cu_k"],
                                c["scale"], c["k_scale"], c["v_scale"], c["cache_dtype"])


def gpu_prefill(pa, c, gpu, waves=0):
    d = cases.to_device(c, gpu)
    out = pa.paged_prefill(d["q"], d["k_cache"], d["v_cache"], d["cu_q"], d["cu_k"], c["max_q"],
                           c["scale"], block_tables=d["block_tables"], k_scale=d["k_scale"],
                           v_scale=d["v_scale"], waves=waves)
    torch.cuda.synchronize()
    return out.cpu()


def check(got, want, kind="fp16"):
    assert not torch.isnan(got).any(), "NaN in the output: a read outside the context"
    rtol, atol = (1e-2, 1e-2) if kind == "fp8" else (1e-3, 2e-3)
    if got.dtype == torch.bfloat16:
        rtol += 2.0 ** -8
    torch.testing.assert_close(got.float(), want.float(), rtol=rtol, atol=atol)


@pytest.fixture(params=[4, 8])
def waves(request):
    """The 4-wave and the 8-wave workgroup shape of the prefill kernel, forced per call."""
    return request.param


def test_config5a_chunked_prefill_bf16_q_fp16_kv(pa, gpu):
    c = make_prefill(1005, [2048] * 8, [512] * 8, 8 * 160 + 32, q_dtype=torch.bfloat16)
    got = gpu_prefill(pa, c, gpu)
    assert got.dtype == torch.bfloat16
    check(got, oracle_prefill(c, upcast=True))


@pytest.mark.parametrize("cache", ["fp16", "fp8", "bf16"])
def test_ragged_chunks(pa, gpu, cache, waves):
    cached = [0, 5, 64, 100, 0, 333, 17]
    new = [1, 63, 64, 65, 200, 7, 130]
    c = make_prefill(60, cached, new, 96, cache=cache)
    # a bf16 cache is exact in the kernel's fp16 (normal range): judged at the 16-bit tolerance, like fp16
    check(gpu_prefill(pa, c, gpu, waves), oracle_prefill(c, upcast=True), "fp8" if cache == "fp8" else "fp16")


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_large_scores_move_the_reference_maximum(pa, gpu, cache, waves):
    """Scores far from zero that grow along the context: the softmax reference that the first key tile sets
    is outgrown by later tiles by more than 2^8, so the lazy rescale of the accumulators runs (a slip there
    is an error of order one).  The kernel rounds the pre-scaled query to fp16 once, which costs 2^-12 of a
    score: at logits of +-40 that is a percent of a probability, so this data is judged at 3e-2, not at the
    1e-3 / 2e-3 of the unit-variance data the path's tolerance is stated for."""
    cached, new = [300, 0, 1000], [100, 260, 64]
    c = make_prefill(66, cached, new, 120, cache=cache)
    c["q"] = (c["q"].float() * 3.5).half()
    bs = c["k_cache"].shape[1]
    # keys grow with their position in the sequence (through the block table, so the ramp follows the context)
    factor = torch.ones(c["k_cache"].shape[0], bs)
    for b, n in enumerate(c["context_lens"].tolist()):
        pos = torch.arange(n)
        factor[c["block_tables"][b, pos // bs].long(), pos % bs] = torch.linspace(0.2, 3.0, n)
    if cache == "fp8":
        c["k_scale"] = c["k_scale"] / factor
    else:
        c["k_cache"] = (c["k_cache"].float() * factor[:, :, None, None]).half()
    got = gpu_prefill(pa, c, gpu, waves)
    assert not torch.isnan(got).any()
    torch.testing.assert_close(got.float(), oracle_prefill(c, upcast=True).float(), rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("hq,hkv,d", [(16, 8, 128), (8, 8, 128), (16, 4, 128), (8, 2, 64), (4, 4, 64)])
def test_head_shapes(pa, gpu, hq, hkv, d, waves):
    c = make_prefill(61 + hq + d, [40, 0, 129], [70, 150, 3], 48, num_heads=hq, num_kv_heads=hkv, head_dim=d)
    check(gpu_prefill(pa, c, gpu, waves), oracle_prefill(c, upcast=True))


@pytest.mark.parametrize("bs", [8, 32, 256])
def test_block_sizes(pa, gpu, bs, waves):
    c = make_prefill(62, [bs * 3 + 1, 0], [100, 77], 64, block_size=bs)
    check(gpu_prefill(pa, c, gpu, waves), oracle_prefill(c, upcast=True))


def test_fp32_query(pa, gpu):
    c = make_prefill(63, [96, 10], [64, 90], 32, q_dtype=torch.float32)
    got = gpu_prefill(pa, c, gpu)
    assert got.dtype == torch.float32
    check(got, oracle_prefill(c))


def test_rows_equal_decode_at_growing_context(pa, gpu):
    # the identity that defines the bottom-right aligned mask: row i == decode at cached + i + 1
    cached, new = 77, 50
    c = make_prefill(64, [cached], [new], 16)
    got = gpu_prefill(pa, c, gpu)
    d = cases.to_device(c, gpu)
    tables = d["block_tables"].expand(new, -1).contiguous()
    lens = torch.arange(cached + 1, cached + new + 1, dtype=torch.int32, device=gpu)
    dec = pa.paged_decode(d["q"], d["k_cache"], d["v_cache"], tables, lens, c["scale"])
    torch.cuda.synchronize()
    torch.testing.assert_close(got.float(), dec.cpu().float(), rtol=1e-3, atol=2e-3)


def test_dense_no_prefix_matches_reference_prefill_fallback(pa, gpu):
    # no cached prefix: K/V are the new tokens themselves (attention.py:281-315)
    g = torch.Generator().manual_seed(65)
    lens = [1, 63, 64, 65, 300]
    total = sum(lens)
    q = torch.randn(total, 16, 128, generator=g).half()
    k = torch.randn(total, 8, 128, generator=g).half()
    v = torch.randn(total, 8, 128, generator=g).half()
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    want = oracle.prefill_no_prefix(q.float(), k.float(), v.float(), cu, cu, 128 ** -0.5)
    got = pa.paged_prefill(q.to(gpu), k.to(gpu), v.to(gpu), cu.to(gpu), cu.to(gpu), max(lens), 128 ** -0.5)
    torch.cuda.synchronize()
    check(got.cpu(), want)
    # bf16 model: q, k, v all bf16
    gotb = pa.paged_prefill(q.bfloat16().to(gpu), k.bfloat16().to(gpu), v.bfloat16().to(gpu), cu.to(gpu),
                            cu.to(gpu), max(lens), 128 ** -0.5)
    torch.cuda.synchronize()
    wantb = oracle.prefill_no_prefix(q.bfloat16().float(), k.bfloat16().float(), v.bfloat16().float(), cu, cu,
                                     128 ** -0.5)
    check(gotb.cpu(), wantb)


def test_module_forward_prefill_then_decode(pa, gpu):
    """PagedAttention.forward: prefill chunk over a cached prefix writes the chunk's K/V and
    attends through the cache; a decode step then continues from it."""
    cached, new = [32, 48], [40, 16]
    c = make_prefill(66, cached, new, 24)
    lens = [a + b for a, b in zip(cached, new)]
    # rebuild the pool holding only the cached part; the module must write the rest
    g = torch.Generator().manual_seed(67)
    k_new = torch.randn(sum(new), 8, 128, generator=g).half()
    v_new = torch.randn(sum(new), 8, 128, generator=g).half()
    slots = []
    for b in range(2):
        pos = torch.arange(cached[b], lens[b])
        slots.append(c["block_tables"][b, pos // 16].long() * 16 + pos % 16)
    slots = torch.cat(slots).to(torch.int32)
    oracle.store_kv_cache(k_new, v_new, c["k_cache"], c["v_cache"], slots)
    want = oracle_prefill(c, upcast=True)
    d = cases.to_device(c, gpu)
    # undo the store on the GPU copy: poison the chunk slots so only the module's write can fill them
    d["k_cache"].view(-1, 8, 128)[slots.long().to(gpu)] = float("nan")
    d["v_cache"].view(-1, 8, 128)[slots.long().to(gpu)] = float("nan")
    attn = pa.PagedAttention(16, 8, 128)
    attn.k_cache, attn.v_cache = d["k_cache"], d["v_cache"]
    pa.set_context(True, cu_seqlens_q=d["cu_q"], cu_seqlens_k=d["cu_k"], max_seqlen_q=max(new),
                   max_seqlen_k=max(lens), slot_mapping=slots.to(gpu), block_tables=d["block_tables"])
    out = attn(d["q"], k_new.to(gpu), v_new.to(gpu))
    pa.reset_context()
    torch.cuda.synchronize()
    check(out.cpu(), want)
    assert torch.equal(d["k_cache"].cpu().view(torch.int16), c["k_cache"].view(torch.int16))


def test_waves_argument_rejects_other_values(lib, gpu):
    t = torch.zeros(64, dtype=torch.float16, device=gpu)
    p = t.data_ptr()
    assert lib.pa_prefill(p, 0, 2048, p, p, None, None, 0, p, 4, p, p, p, 2048, 1, 8, 16, 8, 128, 16, 4, 1.0,
                          6, None) == -1
    assert b"waves_per_workgroup" in lib.pa_last_error()


def test_c_abi_argument_errors(lib, gpu):
    t = torch.zeros(64, dtype=torch.float16, device=gpu)
    p = t.data_ptr()
    def call(d=128, hq=16, hkv=8, kvd=0, bt=p, bs=16, scale=1.0):
        return lib.pa_prefill(p, 0, hq * d, p, p, None, None, kvd, bt, 4, p, p, p, hq * d, 1, 8, hq, hkv,
                              d, bs, 4, scale, 0, None)
    assert call(d=96) == -2
    assert call(hq=15) == -1
    assert call(kvd=3) == -1
    assert call(bs=12) == -2
    assert call(scale=0.0) == -1 and call(scale=-0.1) == -1 and call(scale=float("inf")) == -1
    assert b"scale" in lib.pa_last_error()
