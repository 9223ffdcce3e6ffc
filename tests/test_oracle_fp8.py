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
