"""Pins of oracle/qwen3_block_oracle.py: properties the mathematics fixes, not retyped formulas."""
import math

import torch

from oracle import qwen3_block_oracle as ob


def test_rms_norm_properties():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 3, 128, generator=g)
    y = ob.rms_norm(x, torch.ones(128), 1e-6)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(5, 3), atol=1e-4)
    assert torch.allclose(ob.rms_norm(7.5 * x, torch.ones(128), 1e-12), ob.rms_norm(x, torch.ones(128), 1e-12), atol=1e-5)
    onehot = torch.zeros(1, 1, 64)
    onehot[0, 0, 10] = -3.0
    assert torch.allclose(ob.rms_norm(onehot, torch.ones(64), 0.0)[0, 0, 10], torch.tensor(-8.0))     # -sqrt(64)
    w = torch.arange(1, 129, dtype=torch.float32)
    assert torch.allclose(ob.rms_norm(x, w, 1e-6), y * w, rtol=1e-6, atol=1e-6)
    # the result comes back in the input dtype
    assert ob.rms_norm(x.half(), torch.ones(128).half(), 1e-6).dtype == torch.float16


def test_rotary_properties():
    g = torch.Generator().manual_seed(2)
    d = 128
    f = ob.inv_freq(d)
    assert f[0] == 1.0 and math.isclose(float(f[-1]), 1e6 ** (-(d - 2) / d), rel_tol=1e-5) and f.numel() == d // 2
    x = torch.randn(6, 4, d, generator=g)
    pos = torch.tensor([0, 1, 2, 17, 100, 1000])
    y = ob.apply_rotary_emb(x, pos, f)
    assert torch.equal(y[0], x[0])                                                   # position 0: identity
    pair = lambda t: t[..., : d // 2] ** 2 + t[..., d // 2:] ** 2
    assert torch.allclose(pair(y), pair(x), rtol=1e-5, atol=1e-5)                    # pairs keep their length
    # pair i at position p has turned by p * inv_freq[i] radians
    ang_x = torch.atan2(x[..., d // 2:].double(), x[..., : d // 2].double())
    ang_y = torch.atan2(y[..., d // 2:].double(), y[..., : d // 2].double())
    want = (pos.double()[:, None] * f.double()[None, :])[:, None, :]
    diff = torch.remainder(ang_y - ang_x - want + math.pi, 2 * math.pi) - math.pi
    assert diff.abs().max() < 2e-4        # fp32 cos/sin of angles up to 1000 rad
    # scores depend on the distance between the positions only
    q = torch.randn(1, 1, d, generator=g)
    k = torch.randn(1, 1, d, generator=g)
    score = lambda m, n: (ob.apply_rotary_emb(q, torch.tensor([m]), f) * ob.apply_rotary_emb(k, torch.tensor([n]), f)).sum()
    assert torch.allclose(score(40, 33), score(7, 0), atol=1e-3) and torch.allclose(score(5, 5), (q * k).sum(), atol=1e-4)
    assert not torch.allclose(score(40, 33), score(40, 30), atol=1e-3)
    # 16-bit activations: fp32 inside, optional cast back
    assert ob.apply_rotary_emb(x.half(), pos, f, cast_back=False).dtype == torch.float32
    assert ob.apply_rotary_emb(x.half(), pos, f).dtype == torch.float16


def test_qk_norm_rope_is_the_composition():
    g = torch.Generator().manual_seed(3)
    q, k = torch.randn(4, 16, 128, generator=g).half(), torch.randn(4, 8, 128, generator=g).half()
    qw, kw = (torch.rand(128, generator=g) + 0.5).half(), (torch.rand(128, generator=g) + 0.5).half()
    pos = torch.tensor([3, 9, 27, 81])
    f = ob.inv_freq(128)
    qo, ko = ob.qk_norm_rope(q, k, qw, kw, 1e-6, pos, f)
    assert torch.equal(qo, ob.apply_rotary_emb(ob.rms_norm(q, qw, 1e-6), pos, f))
    assert torch.equal(ko, ob.apply_rotary_emb(ob.rms_norm(k, kw, 1e-6), pos, f))


def test_add_rms_norm_sum_is_correctly_rounded_and_feeds_the_norm():
    g = torch.Generator().manual_seed(21)
    for dt in (torch.float16, torch.bfloat16):
        x = (torch.randn(7, 256, generator=g) * 3).to(dt)
        d = torch.randn(7, 256, generator=g).to(dt)
        w = (torch.rand(256, generator=g) + 0.5).to(dt)
        total, normed = ob.add_rms_norm(x, d, w, 1e-6)
        assert torch.equal(total, (x.double() + d.double()).to(dt))       # one rounding of the exact sum
        assert torch.equal(normed, ob.rms_norm(total, w, 1e-6))


def test_swiglu_closed_forms():
    x = torch.tensor([0.0, 30.0, -30.0, 1.5, -1.5, 0.25, -4.0], dtype=torch.float64)
    one = torch.ones_like(x)
    s = ob.swiglu(x, one)
    assert s[0] == 0 and abs(s[1] - 30.0) < 1e-10 and abs(s[2]) < 1e-10
    torch.testing.assert_close(ob.swiglu(x, one) - ob.swiglu(-x, one), x, rtol=0, atol=1e-12)
    torch.testing.assert_close(s, x * torch.sigmoid(x), rtol=1e-12, atol=1e-12)
    g = torch.Generator().manual_seed(22)
    gate, up = torch.randn(5, 64, generator=g).half(), torch.randn(5, 64, generator=g).half()
    want = ((gate.double() * torch.sigmoid(gate.double())).half().double() * up.double()).half()
    got = ob.swiglu(gate, up)
    assert (got.float() - want.float()).abs().max() <= 2 ** -10 * want.float().abs().max()
