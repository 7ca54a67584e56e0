"""Pins oracle.sample_topk (benchmark.py:58-77) without the reference: special cases that reduce to a
library routine, a brute-force top-k threshold, and the sampling distribution itself."""
import torch

from oracle import ladder_oracle as O


def _logits(B, V, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, V, generator=g) * 3.0


def test_topk_one_is_argmax_whatever_the_noise():
    x = _logits(5, 97, 0)
    noise = torch.empty_like(x).exponential_(1, generator=torch.Generator().manual_seed(1))
    tok, probs = O.sample_topk(x, noise, temperature=0.7, top_k=1)
    assert torch.equal(tok[:, 0].long(), x.argmax(-1))
    assert torch.equal((probs > 0).sum(-1), torch.ones(5, dtype=torch.long))


def test_constant_noise_is_argmax_and_probs_are_softmax():
    x = _logits(4, 64, 2)
    tok, probs = O.sample_topk(x, torch.ones_like(x), temperature=0.8, top_k=None)
    assert torch.equal(tok[:, 0].long(), x.argmax(-1))
    torch.testing.assert_close(probs, torch.softmax(x / 0.8, -1))
    # a cut wider than the vocabulary is no cut
    _, probs_wide = O.sample_topk(x, torch.ones_like(x), temperature=0.8, top_k=10 ** 6)
    assert torch.equal(probs, probs_wide)


def test_temperature_is_clamped():
    x = _logits(2, 32, 3)
    _, p0 = O.sample_topk(x, torch.ones_like(x), temperature=0.0, top_k=None)
    _, p1 = O.sample_topk(x, torch.ones_like(x), temperature=1e-5, top_k=None)
    assert torch.equal(p0, p1)


def test_threshold_matches_a_sort_and_ties_with_the_pivot_stay():
    x = _logits(3, 50, 4)
    x[0, 10:20] = x[0, 5]  # ties
    for k in (1, 7, 11, 50):
        _, probs = O.sample_topk(x, torch.ones_like(x), temperature=1.0, top_k=k)
        for b in range(3):
            vals = sorted(x[b].tolist(), reverse=True)
            pivot = vals[k - 1]
            keep = torch.tensor([v >= pivot for v in x[b].tolist()])
            assert torch.equal(probs[b] > 0, keep)
            ref = torch.softmax(torch.where(keep, x[b], torch.tensor(float("-inf"))), -1)
            torch.testing.assert_close(probs[b], ref)


def test_race_draws_follow_the_probabilities():
    # argmax(p / Exp(1)) picks i with probability p_i: a swapped quotient or a missing cut fails this
    V, N = 6, 200_000
    x = torch.tensor([[2.0, 1.0, 0.0, -1.0, 0.5, 3.0]]).expand(N, V).contiguous()
    noise = torch.empty(N, V).exponential_(1, generator=torch.Generator().manual_seed(5))
    tok, probs = O.sample_topk(x, noise, temperature=1.3, top_k=4)
    freq = torch.bincount(tok[:, 0].long(), minlength=V).double() / N
    assert torch.all(freq[probs[0] == 0] == 0)
    assert (freq - probs[0].double()).abs().max() < 5e-3
