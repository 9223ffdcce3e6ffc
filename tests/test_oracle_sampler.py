"""Pins of oracle/sampler_oracle.py: known distributions, boundaries, frequencies."""
import math

import torch

from oracle import sampler_oracle as so


def logits_for(masses):
    return torch.log(torch.tensor(masses, dtype=torch.float64)).float()[None, :]


def test_top_p_one_is_softmax_and_greedy_is_first_max():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 50, generator=g)
    assert torch.allclose(so.nucleus_probs(x, 0.7, 1.0), torch.softmax(x / 0.7, -1))
    x[1, 7] = x[1, 30] = 9.0
    assert so.greedy(x)[1] == 7


def test_kept_set_on_a_known_distribution():
    masses = [0.05, 0.5, 0.15, 0.3]                      # ranks: 1 (0.5), 3 (0.3), 2 (0.15), 0 (0.05)
    x = logits_for(masses)
    # a token stays iff the mass ranked before it is <= top_p: before = 0, 0.5, 0.8, 0.95
    for top_p, kept in [(0.3, [1]), (0.49, [1]), (0.51, [1, 3]), (0.79, [1, 3]), (0.81, [1, 2, 3]),
                        (0.94, [1, 2, 3]), (0.96, [0, 1, 2, 3])]:
        p = so.nucleus_probs(x, 1.0, top_p)[0]
        assert sorted(torch.nonzero(p > 0).flatten().tolist()) == kept, top_p
        assert math.isclose(float(p.sum()), 1.0, rel_tol=1e-6)
        want = torch.tensor([masses[i] if i in kept else 0.0 for i in range(4)])
        assert torch.allclose(p, want / want.sum(), atol=1e-6)
        assert sorted(torch.nonzero(so.kept_superset(x, 1.0, top_p)[0]).flatten().tolist()) == kept
    # the rule does not depend on where the tokens sit
    perm = torch.tensor([2, 0, 3, 1])
    assert torch.allclose(so.nucleus_probs(x[:, perm], 1.0, 0.6)[0], so.nucleus_probs(x, 1.0, 0.6)[0][perm])


def test_temperature_acts_before_the_cut():
    x = logits_for([0.4, 0.35, 0.25])
    # T = 1: masses ranked before each token 0, 0.4, 0.75
    assert (so.nucleus_probs(x, 1.0, 0.72)[0] > 0).sum() == 2
    # T = 2 flattens to 0.367, 0.343, 0.290: before = 0, 0.367, 0.710 -> the third token now stays
    assert (so.nucleus_probs(x, 2.0, 0.72)[0] > 0).sum() == 3
    # T = 0.1 sharpens to 0.786, 0.207, 0.007: before = 0, 0.786 -> only the first stays
    assert (so.nucleus_probs(x, 0.1, 0.72)[0] > 0).sum() == 1


def test_inverse_cdf_boundaries_and_frequencies():
    probs = torch.tensor([[0.0, 0.5, 0.0, 0.3, 0.2]])
    pick = lambda u: int(so.sample_with_u(probs, torch.tensor([u]))[0])
    assert [pick(0.0), pick(0.4999), pick(0.5001), pick(0.7999), pick(0.8001), pick(0.999999)] == [1, 1, 3, 3, 4, 4]
    g = torch.Generator().manual_seed(2)
    n = 200000
    u = torch.rand(n, generator=g)
    idx = so.sample_with_u(probs.expand(n, -1), u)
    freq = torch.bincount(idx, minlength=5).double() / n
    assert torch.allclose(freq, probs[0].double(), atol=5e-3)
    ref = torch.multinomial(probs[0], n, replacement=True, generator=g)
    freq_ref = torch.bincount(ref, minlength=5).double() / n
    assert torch.allclose(freq, freq_ref, atol=7e-3)


def test_ties_at_the_cut_superset():
    x = torch.tensor([[2.0, 1.0, 1.0, 1.0, 0.0]])
    p = torch.softmax(x.double(), -1)[0]
    top_p = float(p[0] + p[1] * 0.5)                 # the cut falls inside the tie group
    ref = so.nucleus_probs(x, 1.0, top_p)[0] > 0
    sup = so.kept_superset(x, 1.0, top_p)[0]
    assert sup.tolist() == [True, True, True, True, False]
    assert bool((sup | ~ref).all()) and int(ref.sum()) == 2      # the reference keeps part of the group
