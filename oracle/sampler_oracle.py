"""CPU restatement of the reference's token sampler (the parity oracle for pa_sample).

TEST INFRASTRUCTURE ONLY.  Nothing under the product package imports this module; only tests/
do, as the checker.  It follows ModelRunner.sample (src/inference/model_runner.py:590-634):

  greedy            :609-611   argmax over the vocabulary
  nucleus_probs     :613-633   logits.float() / temperature; sort descending, softmax, cumulative
                               sum, mask = cumulative > top_p shifted right by one with the first
                               token always kept; masked logits -> -inf, scattered back; softmax
  sample_with_u     :634       the reference draws with torch.multinomial (its own generator);
                               restated as the inverse-CDF lookup in index order for a given
                               uniform number, which has the same distribution

Pinning (tests/test_oracle_sampler.py):
  * nucleus_probs: top_p = 1 is the plain softmax; a distribution with known masses
    (0.5, 0.3, 0.15, 0.05) keeps exactly the tokens the rule predicts for top_p on either side
    of each cumulative mass; probabilities sum to one and are zero outside the kept set;
    the kept set does not depend on the order of the tokens.
  * sample_with_u: u just below / above each cumulative boundary picks the neighbouring tokens;
    over many uniform numbers the frequencies match nucleus_probs (chi-square), and so do
    torch.multinomial's on the same probabilities, which ties the lookup to the reference's draw.
Ties: torch.sort leaves the order of equal logits unspecified, so when the cut falls inside a
group of equal logits the reference keeps an arbitrary part of the group; `kept_superset` is
the order-free version (all of a tied group stays) that the GPU kernel implements.
"""
import torch


def greedy(logits):
    return torch.argmax(logits, dim=-1)


def nucleus_probs(logits, temperature, top_p):
    scaled = logits.float() / temperature
    if top_p < 1.0:
        sorted_logits, sorted_indices = torch.sort(scaled, descending=True, dim=-1)
        probs = torch.softmax(sorted_logits, dim=-1)
        cumulative = torch.cumsum(probs, dim=-1)
        mask = cumulative > top_p
        mask[..., 1:] = mask[..., :-1].clone()
        mask[..., 0] = False
        sorted_logits[mask] = float("-inf")
        scaled = torch.zeros_like(scaled).scatter_(-1, sorted_indices, sorted_logits)
    return torch.softmax(scaled, dim=-1)


def kept_superset(logits, temperature, top_p):
    """Boolean [B, V]: token j stays iff the softmax mass of the tokens with a strictly larger
    logit is <= top_p.  Equals nucleus_probs > 0 when no two logits at the cut are equal."""
    p = torch.softmax(logits.double() / temperature, dim=-1)
    keep = torch.zeros_like(p, dtype=torch.bool)
    for b in range(p.shape[0]):
        order = torch.argsort(logits[b].double(), descending=True, stable=True)
        lv = logits[b].double()[order]
        csum = torch.cumsum(p[b][order], 0)
        # mass strictly above each token: cumulative mass up to the start of its tie group
        first_of_group = torch.ones_like(lv, dtype=torch.bool)
        first_of_group[1:] = lv[1:] != lv[:-1]
        group_start_mass = torch.where(first_of_group, csum - p[b][order], torch.zeros_like(csum))
        group_start_mass = torch.cummax(group_start_mass, 0).values
        keep[b, order] = group_start_mass <= top_p
    return keep


def sample_with_u(probs, u):
    """First index whose running sum of probs exceeds u (per row); the last kept index if rounding
    leaves u at or above the total."""
    cdf = torch.cumsum(probs.double(), dim=-1)
    target = u.double()[:, None] * cdf[:, -1:]
    hit = cdf > target
    idx = torch.argmax(hit.int(), dim=-1)
    none = ~hit.any(dim=-1)
    if none.any():
        last = (probs > 0).int().cumsum(-1).argmax(-1)
        idx = torch.where(none, last, idx)
    return idx
