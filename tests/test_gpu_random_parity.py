"""Seeded random sweeps of the decode and the chunked-prefill kernels against the oracle.

The other GPU tests pin the benchmark configurations and hand-picked edge cases; these draw the
shape of every case (head layout, block size, batch, context lengths incl. empty rows, table padding,
cache and query dtypes, partition size, launch shape) from a seeded generator, so that combinations
nobody wrote down are exercised too.  Sizes stay small enough for the oracle to take a fraction of
a second per case.  Tolerances are the path's stated ones (rtol 1e-3 / atol 2e-3 for 16-bit caches,
1e-2 / 1e-2 for fp8); bf16 outputs get one extra bf16 rounding on top of the fp32 oracle.
"""
import random

import pytest
import torch

import cases
from oracle import paged_attention_oracle as oracle
from test_gpu_prefill import check as check_prefill, gpu_prefill, make_prefill, oracle_prefill

pytestmark = pytest.mark.gpu


def _tol(cache, out_dtype):
    rtol, atol = (1e-2, 1e-2) if cache == "fp8" else (1e-3, 2e-3)
    if out_dtype == torch.bfloat16:
        rtol += 2.0 ** -8
    return dict(rtol=rtol, atol=atol)


def _decode_case(rng, seed):
    cache = rng.choice(["fp16", "fp16", "fp8", "fp8", "bf16"])
    d = rng.choice([64, 128, 128])
    hkv = rng.choice([1, 2, 4, 8])
    g = rng.choice([1, 2, 2, 3, 4, 8, 16]) if hkv <= 4 else rng.choice([1, 2, 4, 8])
    bs = rng.choice([8, 16, 16, 32, 64])
    batch = rng.choice([1, 2, 3, 5, 8, 13, 33])
    hi = rng.choice([40, 300, 900, 2500]) if hkv * g <= 32 else rng.choice([40, 300])
    lens = [rng.randrange(0 if rng.random() < 0.1 else 1, hi) for _ in range(batch)]
    nb = sum((n + bs - 1) // bs for n in lens) + rng.randrange(1, 9)
    qd = torch.bfloat16 if cache == "bf16" else rng.choice([torch.float16, torch.float16, torch.bfloat16, torch.float32])
    c = cases.make_case(seed, lens, nb, block_size=bs, num_heads=hkv * g, num_kv_heads=hkv, head_dim=d,
                        cache=cache, q_dtype=qd, pad=rng.choice([-1, 0]), extra_cols=rng.randrange(0, 4))
    launch = dict(partition_size=rng.choice([None, None, 16 * rng.randrange(1, 40), 512]),
                  waves=rng.choice([0, 0, 1, 2, 4, 8]))
    return c, lens, cache, launch


@pytest.mark.parametrize("chunk", range(4))
def test_random_decode_cases(pa, gpu, chunk):
    rng = random.Random(9100 + chunk)
    for it in range(12):
        c, lens, cache, launch = _decode_case(rng, 9100 + 100 * chunk + it)
        upcast = c["q"].dtype == torch.bfloat16
        want = oracle.decode(c["q"].float() if upcast else c["q"], c["k_cache"], c["v_cache"], c["block_tables"],
                             c["context_lens"], c["scale"], c["k_scale"], c["v_scale"], c["cache_dtype"])
        dev = cases.to_device(c, gpu)
        try:
            got = pa.paged_decode(dev["q"], dev["k_cache"], dev["v_cache"], dev["block_tables"], dev["context_lens"],
                                  c["scale"], dev["k_scale"], dev["v_scale"], **launch).cpu()
        except RuntimeError as e:
            # a forced wave count that this head layout has no kernel for is refused, not mis-run
            assert launch["waves"] != 0 and "unsupported" in str(e).lower(), (launch, str(e))
            launch["waves"] = 0
            got = pa.paged_decode(dev["q"], dev["k_cache"], dev["v_cache"], dev["block_tables"], dev["context_lens"],
                                  c["scale"], dev["k_scale"], dev["v_scale"], **launch).cpu()
        what = "case %d of chunk %d: cache %s, q %s, shape %s, block %d, lens %s, launch %s" % (
            it, chunk, cache, c["q"].dtype, tuple(c["q"].shape), c["k_cache"].shape[1], lens, launch)
        live = [i for i, n in enumerate(lens) if n > 0]
        empty = [i for i, n in enumerate(lens) if n == 0]
        assert not torch.isnan(got[live]).any(), what
        if live:
            torch.testing.assert_close(got[live].float(), want[live].float(), msg=lambda m: what + "\n" + m,
                                       **_tol(cache, got.dtype))
        if empty:
            assert float(got[empty].float().abs().max()) == 0.0, what


@pytest.mark.parametrize("chunk", range(3))
def test_random_prefill_cases(pa, gpu, chunk):
    rng = random.Random(9500 + chunk)
    for it in range(8):
        cache = rng.choice(["fp16", "fp16", "fp8", "bf16"])
        d = rng.choice([64, 128, 128])
        hkv = rng.choice([1, 2, 4])
        g = rng.choice([1, 2, 3, 4])
        bs = rng.choice([1, 4, 8, 16, 16, 32])
        nseq = rng.choice([1, 2, 3, 5])
        cached = [rng.choice([0, 0, rng.randrange(1, 200), rng.randrange(1, 700)]) for _ in range(nseq)]
        new = [rng.randrange(1, rng.choice([8, 70, 300])) for _ in range(nseq)]
        qd = torch.bfloat16 if cache == "bf16" else rng.choice([torch.float16, torch.bfloat16, torch.float32])
        nb = sum((a + b + bs - 1) // bs for a, b in zip(cached, new)) + rng.randrange(1, 9)
        c = make_prefill(9500 + 100 * chunk + it, cached, new, nb, q_dtype=qd, block_size=bs, num_heads=hkv * g,
                         num_kv_heads=hkv, head_dim=d, cache=cache, pad=rng.choice([-1, 0]))
        waves = rng.choice([0, 4, 8])
        got = gpu_prefill(pa, c, gpu, waves=waves)
        want = oracle_prefill(c, upcast=True)
        try:
            check_prefill(got, want, "fp8" if cache == "fp8" else "fp16")
        except AssertionError as e:
            raise AssertionError("case %d of chunk %d: cache %s, q %s, heads %d/%d x %d, block %d, cached %s, new %s, waves %d\n%s"
                                 % (it, chunk, cache, qd, hkv * g, hkv, d, bs, cached, new, waves, e))
