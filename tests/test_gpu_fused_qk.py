"""Fused per-head q/k RMSNorm + rotary embedding + paged cache write on the GPU.

Floating point: compared with the oracle (the reference's module arithmetic restated on the
CPU, oracle/qwen3_block_oracle.py) within the path's 16-bit tolerance, rtol 1e-3 / atol 2e-3 for
fp16 and fp32, one bf16 rounding (2^-8) more for bf16.  The cache write is byte work on top of
those values: the cache must hold exactly the rotated K the kernel reports and the raw V, and
the fp8 bytes and scales must be exactly what the separate quantising store makes of them.
"""
import pytest
import torch

from oracle import qwen3_block_oracle as ob

pytestmark = pytest.mark.gpu

TOL = {torch.float16: dict(rtol=1e-3, atol=2e-3), torch.float32: dict(rtol=1e-3, atol=2e-3),
       torch.bfloat16: dict(rtol=1e-3 + 2.0 ** -8, atol=1e-2)}


def make(seed, t, hq, hkv, d, dtype, max_pos=4096):
    g = torch.Generator().manual_seed(seed)
    c = dict(q=(2.0 * torch.randn(t, hq, d, generator=g)).to(dtype), k=(0.5 * torch.randn(t, hkv, d, generator=g)).to(dtype),
             v=torch.randn(t, hkv, d, generator=g).to(dtype),
             qw=(torch.rand(d, generator=g) + 0.5).to(dtype), kw=(torch.rand(d, generator=g) + 0.5).to(dtype),
             pos=torch.randint(0, max_pos, (t,), generator=g), inv_freq=ob.inv_freq(d), eps=1e-6)
    c["pos"][0] = 0
    return c


def run(pa, c, gpu, **kw):
    dev = lambda x: x.to(gpu) if isinstance(x, torch.Tensor) else x
    out = pa.qk_norm_rope_store(dev(c["q"]), dev(c["k"]), dev(c["v"]), dev(c["qw"]), dev(c["kw"]), c["eps"],
                                dev(c["inv_freq"]), dev(c["pos"]), **{k: dev(v) for k, v in kw.items()})
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("t,hq,hkv,d", [(64, 16, 8, 128), (5, 8, 8, 128), (33, 8, 2, 64), (1, 4, 4, 64), (600, 16, 8, 128), (515, 4, 2, 64)])
def test_values_against_the_oracle(pa, gpu, dtype, t, hq, hkv, d):
    c = make(70 + t + d, t, hq, hkv, d, dtype)
    q_out, k_out = run(pa, c, gpu, return_k=True)
    want_q, want_k = ob.qk_norm_rope(c["q"], c["k"], c["qw"], c["kw"], c["eps"], c["pos"], c["inv_freq"])
    assert q_out.dtype == dtype and k_out.dtype == dtype
    torch.testing.assert_close(q_out.cpu().float(), want_q.float(), **TOL[dtype])
    torch.testing.assert_close(k_out.cpu().float(), want_k.float(), **TOL[dtype])
    # position 0 is the identity rotation: the row is exactly the rounded norm
    torch.testing.assert_close(q_out[0].cpu().float(), ob.rms_norm(c["q"][:1], c["qw"], c["eps"])[0].float(), **TOL[dtype])


def test_long_positions_keep_their_phase(pa, gpu):
    # 32k-token contexts: the angle reaches 3e4 rad at the fastest frequency
    c = make(71, 16, 16, 8, 128, torch.float16, max_pos=40000)
    c["pos"] = torch.tensor([0, 1, 4095, 4096, 8191, 16384, 20000, 32767, 32768, 39999, 12345, 23456, 31, 777, 9999, 30000])
    q_out, k_out = run(pa, c, gpu, return_k=True)
    want_q, want_k = ob.qk_norm_rope(c["q"], c["k"], c["qw"], c["kw"], c["eps"], c["pos"], c["inv_freq"])
    torch.testing.assert_close(q_out.cpu().float(), want_q.float(), **TOL[torch.float16])
    torch.testing.assert_close(k_out.cpu().float(), want_k.float(), **TOL[torch.float16])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_same_dtype_cache_write_is_the_rotated_k_and_raw_v(pa, gpu, dtype):
    t, hq, hkv, d, nb, bs = 40, 16, 8, 128, 8, 16
    c = make(72, t, hq, hkv, d, dtype)
    g = torch.Generator().manual_seed(5)
    slots = torch.randperm(nb * bs, generator=g)[:t].to(torch.int32)
    slots[3] = -1
    slots[7] = nb * bs + 5            # outside the pool: skipped like a negative slot
    poison = lambda: torch.full((nb, bs, hkv, d), 7.0, dtype=dtype, device=gpu)
    kc, vc = poison(), poison()
    q_out, k_out = run(pa, c, gpu, k_cache=kc, v_cache=vc, slot_mapping=slots, return_k=True)
    want_k, want_v = poison().cpu().view(nb * bs, hkv, d), poison().cpu().view(nb * bs, hkv, d)
    for i, s in enumerate(slots.tolist()):
        if 0 <= s < nb * bs:
            want_k[s] = k_out[i].cpu()
            want_v[s] = c["v"][i]
    assert torch.equal(kc.cpu().view(nb * bs, hkv, d), want_k)
    assert torch.equal(vc.cpu().view(nb * bs, hkv, d), want_v)
    # q does not depend on whether a cache is attached
    assert torch.equal(q_out, run(pa, c, gpu)[0])


@pytest.mark.parametrize("hkv,d", [(8, 128), (2, 64)])
def test_fp8_cache_write_equals_the_separate_quantising_store(pa, gpu, hkv, d):
    t, hq, nb, bs = 37, 2 * hkv, 6, 16
    c = make(73, t, hq, hkv, d, torch.float16)
    c["k"][5] = 0.0                   # an all-zero K row: amax clamps to 1e-5
    slots = torch.randperm(nb * bs, generator=torch.Generator().manual_seed(6))[:t].to(torch.int32)
    slots[11] = -1
    mk = lambda: (torch.zeros(nb, bs, hkv, d, dtype=torch.float8_e4m3fn, device=gpu),
                  torch.zeros(nb, bs, hkv, d, dtype=torch.float8_e4m3fn, device=gpu),
                  torch.ones(nb, bs, device=gpu), torch.ones(nb, bs, device=gpu))
    kc, vc, ks, vs = mk()
    _, k_out = run(pa, c, gpu, k_cache=kc, v_cache=vc, slot_mapping=slots, k_scale=ks, v_scale=vs,
                   cache_dtype="fp8", return_k=True)
    kc2, vc2, ks2, vs2 = mk()
    pa.store_kv_cache(k_out, c["v"].to(gpu), kc2, vc2, slots.to(gpu), ks2, vs2, cache_dtype="fp8")
    torch.cuda.synchronize()
    b = lambda x: x.view(torch.uint8).cpu()
    assert torch.equal(b(kc), b(kc2)) and torch.equal(b(vc), b(vc2))
    assert torch.equal(ks.cpu(), ks2.cpu()) and torch.equal(vs.cpu(), vs2.cpu())


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
@pytest.mark.parametrize("hq,hkv,d", [(16, 8, 128), (6, 2, 64)])
def test_both_launch_shapes_write_the_same_bytes(pa, gpu, cache, hq, hkv, d):
    """Launches of up to 512 tokens run one wave per (token, row group), longer ones one wave per token:
    a chunk of 640 tokens and its two halves must produce the same q, K and cache bytes."""
    t, bs = 640, 16
    nb = t // bs + 3
    c = make(75, t, hq, hkv, d, torch.float16)
    c["k"][17] = 0.0
    slots = torch.randperm(nb * bs, generator=torch.Generator().manual_seed(8))[:t].to(torch.int32)
    slots[5] = -1
    slots[400] = -1
    dev = lambda x: x.to(gpu)

    def pool():
        if cache == "fp8":
            z = lambda: torch.zeros(nb, bs, hkv, d, dtype=torch.float8_e4m3fn, device=gpu)
            return dict(k_cache=z(), v_cache=z(), k_scale=torch.ones(nb, bs, device=gpu), v_scale=torch.ones(nb, bs, device=gpu),
                        cache_dtype="fp8")
        z = lambda: torch.full((nb, bs, hkv, d), 3.0, dtype=torch.float16, device=gpu)
        return dict(k_cache=z(), v_cache=z())

    def call(lo, hi, kw):
        return pa.qk_norm_rope_store(dev(c["q"][lo:hi]), dev(c["k"][lo:hi]), dev(c["v"][lo:hi]), dev(c["qw"]), dev(c["kw"]),
                                     c["eps"], dev(c["inv_freq"]), dev(c["pos"][lo:hi]), slot_mapping=dev(slots[lo:hi]),
                                     return_k=True, **kw)

    whole, halves = pool(), pool()
    q1, k1 = call(0, t, whole)
    parts = [call(0, t // 2, halves), call(t // 2, t, halves)]
    torch.cuda.synchronize()
    assert torch.equal(q1, torch.cat([p[0] for p in parts])) and torch.equal(k1, torch.cat([p[1] for p in parts]))
    for name in whole:
        if name != "cache_dtype":
            a, b = whole[name], halves[name]
            assert torch.equal(a.view(torch.uint8) if a.dtype == torch.float8_e4m3fn else a,
                               b.view(torch.uint8) if b.dtype == torch.float8_e4m3fn else b), name


def test_packed_qkv_views_and_errors(pa, lib, gpu):
    t, hq, hkv, d = 9, 16, 8, 128
    c = make(74, t, hq, hkv, d, torch.float16)
    packed = torch.cat([c["q"].reshape(t, -1), c["k"].reshape(t, -1), c["v"].reshape(t, -1)], dim=1).to(gpu)
    qv = packed[:, :hq * d].view(t, hq, d)
    kv = packed[:, hq * d:(hq + hkv) * d].view(t, hkv, d)
    vv = packed[:, (hq + hkv) * d:].view(t, hkv, d)
    kc = torch.zeros(2, 16, hkv, d, dtype=torch.float16, device=gpu)
    vc = torch.zeros_like(kc)
    slots = torch.arange(t, dtype=torch.int32, device=gpu)
    dev = lambda x: x.to(gpu)
    got = pa.qk_norm_rope_store(qv, kv, vv, dev(c["qw"]), dev(c["kw"]), c["eps"], dev(c["inv_freq"]), dev(c["pos"]),
                                k_cache=kc, v_cache=vc, slot_mapping=slots, return_k=True)
    ref = run(pa, c, gpu, return_k=True)
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    assert torch.equal(kc.view(-1, hkv, d)[:t], ref[1]) and torch.equal(vc.view(-1, hkv, d)[:t], dev(c["v"]))
    with pytest.raises(RuntimeError, match="no CPU path"):
        pa.qk_norm_rope_store(c["q"], c["k"], c["v"], c["qw"], c["kw"], c["eps"], c["inv_freq"], c["pos"])
    with pytest.raises(RuntimeError, match="inv_freq"):
        pa.qk_norm_rope_store(qv, kv, vv, dev(c["qw"]), dev(c["kw"]), c["eps"], dev(c["inv_freq"])[:10], dev(c["pos"]))
    # C ABI: unsupported head_dim
    rc = lib.pa_qk_norm_rope_store(qv.data_ptr(), kv.data_ptr(), None, 0, 96, 96, 0, c["qw"].to(gpu).data_ptr(),
                                   c["kw"].to(gpu).data_ptr(), 0, 1e-6, dev(c["inv_freq"]).data_ptr(),
                                   dev(c["pos"]).data_ptr(), qv.data_ptr(), 96, None, 0, None, None, None, None, 0,
                                   None, 1, 1, 1, 96, 0, None)
    assert rc != 0 and b"head_dim" in lib.pa_last_error()
