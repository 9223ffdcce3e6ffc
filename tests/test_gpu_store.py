"""Paged KV-cache write on the GPU against the oracle: bit-exact cache bytes and scales."""
import numpy as np
import pytest
import torch

from oracle import e4m3fn
from oracle import paged_attention_oracle as oracle

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _slots(gen, n, total, skip_every=5):
    s = torch.randperm(total, generator=gen)[:n].to(torch.int32)
    s[::skip_every] = -1
    return s


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,hkv,d", [(64, 8, 128), (1, 8, 128), (257, 2, 64), (33, 4, 128)])
def test_fp16_store_bit_exact(pa, gpu, dtype, n, hkv, d):
    g = torch.Generator().manual_seed(n * 7 + d)
    nb, bs = 40, 16
    k = torch.randn(n, hkv, d, generator=g).to(dtype)
    v = torch.randn(n, hkv, d, generator=g).to(dtype)
    slots = _slots(g, n, nb * bs)
    kc = torch.randn(nb, bs, hkv, d, generator=g).to(dtype)
    vc = torch.randn(nb, bs, hkv, d, generator=g).to(dtype)
    kc_g, vc_g = kc.to(gpu), vc.to(gpu)
    oracle.store_kv_cache(k, v, kc, vc, slots)
    pa.store_kv_cache(k.to(gpu), v.to(gpu), kc_g, vc_g, slots.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(kc_g.cpu().view(torch.uint8), kc.view(torch.uint8))
    assert torch.equal(vc_g.cpu().view(torch.uint8), vc.view(torch.uint8))


def test_fp16_store_strided_input_and_out_of_range_slots(pa, gpu):
    g = torch.Generator().manual_seed(5)
    nb, bs, hkv, d = 8, 16, 8, 128
    qkv = torch.randn(20, (16 + 2 * hkv) * d, generator=g).half()
    k = qkv[:, 16 * d:(16 + hkv) * d].view(20, hkv, d)          # non-contiguous token stride
    v = qkv[:, (16 + hkv) * d:].view(20, hkv, d)
    slots = torch.arange(20, dtype=torch.int32) * 3
    slots[3] = -1
    slots[7] = -5
    kc = torch.zeros(nb, bs, hkv, d, dtype=torch.float16)
    vc = torch.zeros(nb, bs, hkv, d, dtype=torch.float16)
    kc_g, vc_g = kc.to(gpu), vc.to(gpu)
    oracle.store_kv_cache(k, v, kc, vc, slots)
    qkv_g = qkv.to(gpu)
    kg = qkv_g[:, 16 * d:(16 + hkv) * d].view(20, hkv, d)
    vg = qkv_g[:, (16 + hkv) * d:].view(20, hkv, d)
    big = slots.clone()
    big[11] = nb * bs + 4          # beyond the pool: skipped on the GPU (the host path would raise)
    ref_k, ref_v = kc.clone(), vc.clone()
    ref_k.view(-1, hkv, d)[int(slots[11])] = 0
    ref_v.view(-1, hkv, d)[int(slots[11])] = 0
    pa.store_kv_cache(kg, vg, kc_g, vc_g, big.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(kc_g.cpu(), ref_k) and torch.equal(vc_g.cpu(), ref_v)


def _fp8_roundtrip(pa, gpu, k, v, slots, nb, bs):
    hkv, d = k.shape[1], k.shape[2]
    kc = torch.zeros(nb, bs, hkv, d, dtype=FP8)
    vc = torch.zeros(nb, bs, hkv, d, dtype=FP8)
    kc.view(torch.uint8).fill_(0x11)
    vc.view(torch.uint8).fill_(0x22)
    ks = torch.full((nb, bs), 7.0)
    vs = torch.full((nb, bs), 9.0)
    kc_g, vc_g, ks_g, vs_g = kc.to(gpu), vc.to(gpu), ks.to(gpu), vs.to(gpu)
    oracle.store_kv_cache(k, v, kc, vc, slots, ks, vs, "fp8")
    pa.store_kv_cache(k.to(gpu), v.to(gpu), kc_g, vc_g, slots.to(gpu), ks_g, vs_g, "fp8")
    torch.cuda.synchronize()
    assert torch.equal(ks_g.cpu().view(torch.int32), ks.view(torch.int32)), "k scales differ"
    assert torch.equal(vs_g.cpu().view(torch.int32), vs.view(torch.int32)), "v scales differ"
    assert torch.equal(kc_g.cpu().view(torch.uint8), kc.view(torch.uint8)), "k bytes differ"
    assert torch.equal(vc_g.cpu().view(torch.uint8), vc.view(torch.uint8)), "v bytes differ"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,hkv,d", [(64, 8, 128), (4096, 8, 128), (3, 2, 64), (19, 16, 128), (5, 32, 128)])
def test_fp8_store_bit_exact_random(pa, gpu, dtype, n, hkv, d):
    g = torch.Generator().manual_seed(n + hkv)
    nb, bs = (n + 15) // 16 + 3, 16
    # token magnitudes spread over many binades so that many different scales are exercised
    mag = torch.exp(torch.randn(n, 1, 1, generator=g) * 3)
    k = (torch.randn(n, hkv, d, generator=g) * mag).to(dtype)
    v = (torch.randn(n, hkv, d, generator=g) * mag.flip(0)).to(dtype)
    _fp8_roundtrip(pa, gpu, k, v, _slots(g, n, nb * bs, skip_every=7), nb, bs)


def test_fp8_store_edge_rows(pa, gpu):
    hkv, d = 8, 128
    rows = []
    z = torch.zeros(hkv * d)
    rows.append(z.clone())                                   # all zero: amax clamps to 1e-5
    r = z.clone(); r[0] = -0.0; r[1] = 1e-7; r[2] = -1e-6; rows.append(r)   # below the clamp
    r = z.clone(); r[0] = 448.0; r[1] = 1.0 * 2 ** -10; r[2] = 3.0 * 2 ** -10; r[3] = -2.0 ** -9
    r[4] = 7.5 * 2 ** -9; r[5] = 1.0625; r[6] = 1.1875; r[7] = -0.0; rows.append(r)   # scale == 1: ties
    r = torch.linspace(-3, 3, hkv * d); rows.append(r)
    r = z.clone(); r[5] = 65504.0; r[6] = 6e-8; r[7] = -65504.0; rows.append(r)   # fp16 extremes
    r = z.clone(); r[100] = 2.0 ** -14; rows.append(r)
    k = torch.stack(rows).view(-1, hkv, d).half()
    v = torch.flip(k, dims=[0]).contiguous()
    slots = torch.arange(k.shape[0], dtype=torch.int32) * 2
    _fp8_roundtrip(pa, gpu, k, v, slots, 4, 16)


def test_fp8_store_every_finite_fp16_pattern(pa, gpu):
    bits = np.arange(65536, dtype=np.uint16)
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.float16)
    x = x[torch.isfinite(x)]
    pad = (-x.numel()) % 1024
    x = torch.cat([x, torch.zeros(pad, dtype=torch.float16)])
    g = torch.Generator().manual_seed(3)
    x = x[torch.randperm(x.numel(), generator=g)]
    k = x.view(-1, 8, 128)
    v = x.flip(0).view(-1, 8, 128).contiguous()
    n = k.shape[0]
    _fp8_roundtrip(pa, gpu, k, v, torch.arange(n, dtype=torch.int32), (n + 15) // 16, 16)


def test_f32_to_fp8_converter_matches_torch_and_numpy(lib, gpu):
    g = torch.Generator().manual_seed(9)
    x = torch.randn(1 << 20, generator=g) * torch.exp(torch.randn(1 << 20, generator=g) * 4)
    special = torch.tensor([0.0, -0.0, 448.0, 464.0, 465.0, 479.9, 480.0, 1e9, float("inf"),
                            -float("inf"), 2.0 ** -9, 2.0 ** -10, 3 * 2.0 ** -10, 2.0 ** -6, 1e-30])
    x = torch.cat([x, special, -special])
    xg = x.to(gpu)
    out = torch.empty(x.numel(), dtype=torch.uint8, device=gpu)
    assert lib.pa_f32_to_fp8_e4m3(xg.data_ptr(), out.data_ptr(), x.numel(), None) == 0
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.array_equal(got, x.to(FP8).view(torch.uint8).numpy())
    assert np.array_equal(got, e4m3fn.encode(x.numpy()))


def test_fp8_to_f32_converter_all_codes(lib, gpu):
    codes = torch.arange(256, dtype=torch.uint8)
    out = torch.empty(256, dtype=torch.float32, device=gpu)
    cg = codes.to(gpu)
    assert lib.pa_fp8_e4m3_to_f32(cg.data_ptr(), out.data_ptr(), 256, None) == 0
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    want = e4m3fn.decode(codes.numpy())
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])


def test_store_rejects_mismatched_arguments(pa, gpu):
    k = torch.zeros(2, 8, 128, dtype=torch.float16, device=gpu)
    cache = torch.zeros(4, 16, 8, 128, dtype=torch.float16, device=gpu)
    slots = torch.zeros(2, dtype=torch.int32, device=gpu)
    with pytest.raises(RuntimeError):
        pa.store_kv_cache(k.bfloat16(), k.bfloat16(), cache, cache.clone(), slots)
    with pytest.raises(RuntimeError):
        pa.store_kv_cache(k, k, cache.to(FP8), cache.to(FP8), slots, cache_dtype="fp8")   # no scales
    with pytest.raises(RuntimeError):
        pa.store_kv_cache(k[:, :4], k[:, :4], cache, cache.clone(), slots)
    pa.store_kv_cache(k[:0], k[:0], cache, cache.clone(), slots[:0])                       # empty: no-op
