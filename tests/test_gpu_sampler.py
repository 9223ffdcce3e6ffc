"""pa_sample on the GPU against the oracle (oracle/sampler_oracle.py).

Index work: greedy must equal argmax exactly (first maximum).  The sampled index, for a given
uniform number, must equal the oracle's inverse-CDF lookup over the oracle's kept set; rows whose
uniform number falls within 5e-6 of a cumulative boundary (where fp32 summation order decides)
are excluded from the exact comparison and must land between the tokens the oracle picks for
u - 2e-5 and u + 2e-5.
"""
import pytest
import torch

from oracle import sampler_oracle as so

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("vocab", [151936, 1000, 65, 1])
def test_greedy_is_the_first_maximum(pa, gpu, dtype, vocab):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(16, vocab, generator=g).to(dtype)
    if vocab > 10:
        x[2, 5] = x[2, vocab - 3] = 30.0           # tie: the first wins
        x[3, :] = -float("inf")
        x[3, vocab // 2] = -5.0
    got = pa.sample_tokens(x.to(gpu), temperature=0.0)
    assert got.dtype == torch.int64 and torch.equal(got.cpu(), so.greedy(x.float()))
    # a strided view (logits of the last position of each sequence)
    wide = torch.zeros(16, vocab + 8, dtype=dtype)
    wide[:, :vocab] = x
    assert torch.equal(pa.sample_tokens(wide.to(gpu)[:, :vocab], temperature=-1.0).cpu(), so.greedy(x.float()))


def check_against_oracle(pa, gpu, x, temperature, top_p, seed):
    b = x.shape[0]
    u = torch.rand(b, generator=torch.Generator().manual_seed(seed))
    got = pa.sample_tokens(x.to(gpu), temperature, top_p, uniforms=u.to(gpu)).cpu()
    keep = so.kept_superset(x.float(), temperature, top_p)
    p = torch.softmax(x.double() / temperature, -1) * keep
    p = p / p.sum(-1, keepdim=True)
    want = so.sample_with_u(p, u)
    cdf = torch.cumsum(p, -1)
    margin = (cdf - u.double()[:, None]).abs().min(-1).values
    safe = margin > 5e-6
    assert safe.float().mean() > 0.5
    assert torch.equal(got[safe], want[safe])
    assert bool(keep[torch.arange(b), got].all()), "a token outside the nucleus was drawn"
    # near a boundary either neighbour is acceptable
    for r in torch.nonzero(~safe).flatten().tolist():
        lo = so.sample_with_u(p[r:r + 1], (u[r:r + 1] - 2e-5).clamp(min=0))
        hi = so.sample_with_u(p[r:r + 1], (u[r:r + 1] + 2e-5).clamp(max=0.999999))
        assert int(lo) <= int(got[r]) <= int(hi)
    return got, keep


@pytest.mark.parametrize("temperature,top_p", [(0.7, 0.9), (1.0, 0.5), (1.3, 1.0), (0.3, 0.99)])
def test_fp32_rows_match_the_oracle_draw(pa, gpu, temperature, top_p):
    g = torch.Generator().manual_seed(4)
    x = 3.0 * torch.randn(64, 4096, generator=g)
    got, keep = check_against_oracle(pa, gpu, x, temperature, top_p, 5)
    if top_p < 1.0:
        # without ties the order-free kept set is the reference's
        ref_keep = so.nucleus_probs(x, temperature, top_p) > 0
        assert torch.equal(keep, ref_keep)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_sixteen_bit_rows_with_ties_at_vocabulary_size(pa, gpu, dtype):
    g = torch.Generator().manual_seed(6)
    x = (2.5 * torch.randn(8, 151936, generator=g)).to(dtype)       # thousands of equal logits per row
    check_against_oracle(pa, gpu, x, 0.7, 0.9, 7)


def test_frequencies_follow_the_nucleus_distribution(pa, gpu):
    masses = torch.tensor([0.02, 0.4, 0.08, 0.3, 0.2])
    x = torch.log(masses)[None, :].expand(50000, -1).contiguous()
    got = pa.sample_tokens(x.to(gpu), 1.0, 0.85, generator=torch.Generator(device=gpu).manual_seed(8)).cpu()
    want = so.nucleus_probs(x[:1], 1.0, 0.85)[0]                     # keeps 0.4, 0.3, 0.2 (before = 0, 0.4, 0.7), drops the rest
    assert (want > 0).tolist() == [False, True, False, True, True]
    freq = torch.bincount(got, minlength=5).double() / got.numel()
    assert torch.allclose(freq, want.double(), atol=1e-2)


def test_model_runner_sample_and_errors(pa, lib, gpu):
    runner = pa.ModelRunner(None, pa.ModelRunnerConfig())
    x = torch.randn(4, 100, generator=torch.Generator().manual_seed(9))
    assert runner.sample(x.to(gpu), temperature=0) == so.greedy(x).tolist()
    ids = runner.sample(x.to(gpu), temperature=0.7, top_p=0.9)
    assert isinstance(ids, list) and len(ids) == 4 and all(0 <= i < 100 for i in ids)
    with pytest.raises(RuntimeError, match="no CPU path"):
        pa.sample_tokens(x)
    with pytest.raises(RuntimeError, match="uniforms"):
        pa.sample_tokens(x.to(gpu), 0.7, 0.9, uniforms=torch.rand(3, device=gpu))
    out = torch.zeros(4, dtype=torch.int64, device=gpu)
    assert lib.pa_sample(x.to(gpu).data_ptr(), 2, 100, 4, 100, 0.7, 0.9, None, out.data_ptr(), None) != 0
    assert b"uniform" in lib.pa_last_error()
    assert lib.pa_sample(x.to(gpu).data_ptr(), 2, 50, 4, 100, 0.0, 0.9, None, out.data_ptr(), None) != 0
