"""Pins the fp8-e4m3fn cast the oracle relies on (torch's .to(float8_e4m3fn), the call the
reference makes at src/inference/attention.py:109-110) and the oracle's quantising store."""
import json
import os

import numpy as np
import torch

from oracle import e4m3fn
from oracle import paged_attention_oracle as oracle

HERE = os.path.dirname(os.path.abspath(__file__))


def _kat():
    with open(os.path.join(HERE, "golden", "e4m3fn_kat.json")) as f:
        return [(float(v), b) for v, b in json.load(f)["vectors"]]


def test_kat_numpy_encoder():
    for value, byte in _kat():
        got = int(e4m3fn.encode(np.array([value], dtype=np.float32))[0])
        assert got == byte, (value, got, byte)


def test_kat_torch_cast():
    for value, byte in _kat():
        got = int(torch.tensor([value], dtype=torch.float32).to(torch.float8_e4m3fn).view(torch.uint8)[0])
        assert got == byte, (value, got, byte)


def test_torch_cast_equals_numpy_encoder_on_every_fp16_pattern():
    bits = np.arange(65536, dtype=np.uint16)
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.float16).float()
    for s in (1.0, 448.0 / 3.7, 0.013, 100.0, 448.0 / 65504.0):
        y = x * s
        want = e4m3fn.encode(y.numpy())
        got = y.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(want, got)


def test_decode_table_matches_torch():
    b = torch.arange(256, dtype=torch.uint8)
    want = b.view(torch.float8_e4m3fn).float().numpy()
    got = e4m3fn.decode(b.numpy())
    assert np.array_equal(np.isnan(want), np.isnan(got))
    assert np.array_equal(want[~np.isnan(want)], got[~np.isnan(got)])


def test_decode_encode_roundtrip_is_identity_on_finite_codes():
    codes = np.array([c for c in range(256) if c not in (0x7F, 0xFF)], dtype=np.uint8)
    assert np.array_equal(e4m3fn.encode(e4m3fn.decode(codes)), codes)


def test_quantize_per_token_closed_form():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(5, 8, 128, generator=g).half()
    x[3] = 0                                   # all-zero token: amax clamps to 1e-5
    q, s = oracle.quantize_fp8_per_token(x)
    for t in range(5):
        amax = max(float(x[t].float().abs().max()), 1e-5)
        # python-scalar / tensor is reciprocal-then-multiply in torch (two fp32 roundings)
        want_s = (np.float32(1.0) / np.float32(amax)) * np.float32(448.0)
        assert np.float32(s[t]) == want_s
        y = x[t].float().numpy().astype(np.float32) * want_s
        assert np.array_equal(e4m3fn.encode(y), q[t].view(torch.uint8).numpy())
    assert float(s[3]) == float((np.float32(1.0) / np.float32(1e-5)) * np.float32(448.0))
    assert int(q[3].view(torch.uint8).max()) == 0
    # the largest element of a token always lands on +-448
    for t in (0, 1, 2, 4):
        assert int((q[t].view(torch.uint8) & 0x7F).max()) == 0x7E


def test_fp8_store_scatter_and_untouched_slots():
    g = torch.Generator().manual_seed(8)
    nb, bs, h, d = 6, 16, 2, 64
    k = torch.randn(10, h, d, generator=g).half()
    v = torch.randn(10, h, d, generator=g).half()
    kc = torch.zeros(nb, bs, h, d, dtype=torch.float8_e4m3fn)
    vc = torch.zeros(nb, bs, h, d, dtype=torch.float8_e4m3fn)
    kc.view(torch.uint8).fill_(0x55)
    vc.view(torch.uint8).fill_(0x55)
    ks = torch.full((nb, bs), 3.0)
    vs = torch.full((nb, bs), 3.0)
    slots = torch.tensor([5, -1, 17, 95, 0, -1, 33, 34, 35, 64], dtype=torch.int32)
    oracle.store_kv_cache(k, v, kc, vc, slots, ks, vs, "fp8")
    kq, s = oracle.quantize_fp8_per_token(k)
    touched = set()
    for t, sl in enumerate(slots.tolist()):
        if sl < 0:
            continue
        touched.add(sl)
        assert torch.equal(kc.view(-1, h, d)[sl].view(torch.uint8), kq[t].view(torch.uint8))
        assert float(ks.view(-1)[sl]) == float(s[t])
    for sl in range(nb * bs):
        if sl not in touched:
            assert int(kc.view(-1, h, d)[sl].view(torch.uint8).min()) == 0x55
            assert float(vs.view(-1)[sl]) == 3.0


def _store_and_dequant(x):
    """x [N, H, D] fp16 -> what a reader of the fp8 cache sees: the oracle's store followed by the
    oracle's gather (fp8 -> fp16 -> divide by the token's scale, attention.py:355-362)."""
    n, h, d = x.shape
    nb = (n + 15) // 16
    kc = torch.zeros(nb, 16, h, d, dtype=torch.float8_e4m3fn)
    vc = torch.zeros(nb, 16, h, d, dtype=torch.float8_e4m3fn)
    ks, vs = torch.ones(nb, 16), torch.ones(nb, 16)
    slots = torch.arange(n, dtype=torch.int32)
    oracle.store_kv_cache(x, x, kc, vc, slots, ks, vs, "fp8")
    ki, vi = oracle._gather_kv(kc, vc, slots.long(), ks, vs, True)
    assert ki.dtype == torch.float32 and torch.equal(ki, vi)
    return ki, ks.view(-1)[:n]


def test_dequant_of_quant_stays_within_half_an_e4m3_step_of_the_source():
    """What is read back differs from what was written by at most half a step of the e4m3 grid at
    that magnitude: 2^-4 relative for normal codes (3 mantissa bits), 2^-10 / scale absolute in the
    subnormal range (grid 2^-9 below 2^-6), element by element.  A dequant that multiplied by the
    scale, used the wrong token's scale or dropped it fails by orders of magnitude."""
    g = torch.Generator().manual_seed(21)
    rows = [torch.randn(40, 8, 128, generator=g),
            torch.randn(8, 8, 128, generator=g) * torch.logspace(-4, 3, 8)[:, None, None],   # tokens of very different size
            torch.zeros(1, 8, 128)]
    edge = torch.zeros(3, 8, 128)
    edge[0, 0, 0] = 60000.0                      # one huge element: everything else lands in the subnormals
    edge[0, 1, :] = torch.linspace(-1.0, 1.0, 128)
    edge[1, :, :] = 2.0 ** -14                   # fp16's smallest normal everywhere
    edge[2, 3, 5] = -0.0
    x = torch.cat(rows + [edge]).half()
    back, s = _store_and_dequant(x)
    xf = x.float()
    step = torch.maximum(xf.abs() * 2.0 ** -4, (2.0 ** -10 / s)[:, None, None])
    assert torch.all((back - xf).abs() <= step * (1 + 2.0 ** -20))
    # the bound is tight somewhere (the test would notice a quantiser with more bits than e4m3)
    assert float(((back - xf).abs() / step).max()) > 0.9
    # and the largest element of every non-zero token comes back within the fp32 scale rounding
    amax = xf.abs().amax(dim=(1, 2))
    nz = amax > 0
    assert torch.allclose(back.abs().amax(dim=(1, 2))[nz], amax[nz], rtol=2.0 ** -20)


def test_fp8_cache_decode_tracks_fp16_cache_decode_of_the_same_source():
    """The same K/V written through the fp16 store and through the fp8 store decode to outputs that
    differ by quantisation noise only.  For N(0,1) data an e4m3 element carries about 2^-4 / sqrt(3)
    relative error; over head_dim 128 that gives score errors of about 0.04 and output errors of a few
    percent of the output scale.  Bound used: 8e-2 absolute, 6e-2 of the Frobenius norm."""
    g = torch.Generator().manual_seed(22)
    lens, nb, bs, hq, hkv, d = [37, 200, 512], 64, 16, 16, 8, 128
    need = [(n + bs - 1) // bs for n in lens]
    perm = torch.randperm(nb, generator=g)
    tables = torch.full((3, max(need)), -1, dtype=torch.int32)
    caches = {"fp16": (torch.zeros(nb, bs, hkv, d, dtype=torch.float16), torch.zeros(nb, bs, hkv, d, dtype=torch.float16),
                       None, None),
              "fp8": (torch.zeros(nb, bs, hkv, d, dtype=torch.float8_e4m3fn),
                      torch.zeros(nb, bs, hkv, d, dtype=torch.float8_e4m3fn), torch.ones(nb, bs), torch.ones(nb, bs))}
    cur = 0
    for b, n in enumerate(lens):
        tables[b, :need[b]] = perm[cur:cur + need[b]].to(torch.int32)
        cur += need[b]
        k = torch.randn(n, hkv, d, generator=g).half()
        v = torch.randn(n, hkv, d, generator=g).half()
        pos = torch.arange(n)
        slots = (tables[b, pos // bs].long() * bs + pos % bs).to(torch.int32)
        for kind, (kc, vc, ks, vs) in caches.items():
            oracle.store_kv_cache(k, v, kc, vc, slots, ks, vs, kind)
    q = torch.randn(3, hq, d, generator=g)
    lens_t = torch.tensor(lens, dtype=torch.int32)
    out = {kind: oracle.decode(q, kc.float() if kind == "fp16" else kc, vc.float() if kind == "fp16" else vc,
                               tables, lens_t, d ** -0.5, ks, vs, kind)
           for kind, (kc, vc, ks, vs) in caches.items()}
    diff = (out["fp8"] - out["fp16"]).abs()
    assert 1e-4 < float(diff.max()) < 8e-2
    assert float(diff.norm() / out["fp16"].norm()) < 6e-2
