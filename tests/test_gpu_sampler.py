"""lr_sample_topk through the C ABI against oracle.sample_topk on the same bf16 logits and the same
Exp(1) draws.  Integer work is exact: the set of kept tokens (the top-k cut) and the token that wins
the race given the kernel's own probabilities.  Probabilities are floating point: the softmax sum is
accumulated in a different order than torch's, tolerance one bf16 step."""
import pytest
import torch

from oracle import ladder_oracle as O

pytestmark = pytest.mark.gpu


def _hip():
    import os
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                                    "ladder-residual-inference_amd"))
    from gpt_fast import _hip
    return _hip


def _ulp_diff(a, b):
    return (a.view(torch.int16).int() - b.view(torch.int16).int()).abs()


CASES = [
    # B, V, ld, temperature, top_k
    (1, 256, 256, 0.8, 200),
    (3, 1000, 1008, 0.8, 200),      # V not a multiple of 8, rows inside a wider buffer
    (2, 16032, 16032, 0.8, 200),    # the vocabulary shard of the TP = 8 configurations
    (1, 128256, 128256, 1.0, 200),  # full vocabulary
    (2, 16032, 16032, 0.8, None),   # no cut
    (2, 512, 512, 0.8, 100000),     # cut wider than the row
    (4, 4096, 4096, 1e-7, 50),      # temperature below the clamp
    (2, 2048, 2048, 1.5, 1),        # top-1
]


@pytest.mark.parametrize("B,V,ld,temperature,top_k", CASES)
def test_sample_topk_matches_oracle(B, V, ld, temperature, top_k):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(1234 + V)
    buf = (torch.randn(B, ld, device="cuda", generator=g) * 4.0).to(torch.bfloat16)
    logits = buf[:, :V]
    noise = torch.empty(B, V, device="cuda", dtype=torch.bfloat16).exponential_(1, generator=g)
    ref_tok, ref_probs = O.sample_topk(logits, noise, temperature, top_k)
    out = torch.full((B, 1), -1, dtype=torch.int32, device="cuda")
    probs = torch.full((B, V), 7.0, dtype=torch.bfloat16, device="cuda")
    hip.sample_topk(logits, noise, temperature, top_k, out, probs)
    torch.cuda.synchronize()
    # the top-k cut is integer work: exactly the same tokens survive
    assert torch.equal(probs > 0, ref_probs > 0)
    assert int(_ulp_diff(probs, ref_probs).max()) <= 1
    # the race given the kernel's own probabilities: exact, lowest index among equals
    own = torch.argmax(probs / noise, dim=-1, keepdim=True).to(torch.int32)
    assert torch.equal(out, own)
    # rows whose probabilities agree bit for bit must give the oracle's token
    same = (probs.view(torch.int16) == ref_probs.view(torch.int16)).all(dim=-1)
    assert torch.equal(out[same], ref_tok[same])


def test_sample_topk_ties_and_minus_inf():
    hip = _hip()
    V = 777
    logits = torch.zeros(2, V, device="cuda", dtype=torch.bfloat16)
    logits[0, 100:400] = 2.0            # 300 equal maxima: more than top_k survive the cut
    logits[1, :] = float("-inf")
    logits[1, 5] = 1.0
    logits[1, 9] = 1.0
    noise = torch.ones(2, V, device="cuda", dtype=torch.bfloat16)
    noise[1, 9] = 0.5                   # the second of the two survivors wins the race
    ref_tok, ref_probs = O.sample_topk(logits, noise, 0.8, 200)
    out = torch.empty(2, 1, dtype=torch.int32, device="cuda")
    probs = torch.empty(2, V, dtype=torch.bfloat16, device="cuda")
    hip.sample_topk(logits, noise, 0.8, 200, out, probs)
    torch.cuda.synchronize()
    assert int((probs[0] > 0).sum()) == 300 and torch.equal(probs > 0, ref_probs > 0)
    assert int(_ulp_diff(probs, ref_probs).max()) <= 1
    assert out[0, 0].item() == 100 and out[1, 0].item() == 9
    assert torch.equal(out, ref_tok)


def test_sample_topk_without_probs_and_errors():
    hip = _hip()
    logits = (torch.randn(2, 640, device="cuda") * 3).to(torch.bfloat16)
    noise = torch.empty_like(logits).exponential_(1)
    out = torch.empty(2, 1, dtype=torch.int32, device="cuda")
    probs = torch.empty_like(logits)
    hip.sample_topk(logits, noise, 0.8, 200, out, probs)
    out2 = torch.empty_like(out)
    hip.sample_topk(logits, noise, 0.8, 200, out2, None)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    lib = hip.load()
    assert lib.lr_sample_topk(None, 640, noise.data_ptr(), 640, 2, 640, 0.8, 200, None, 0, out.data_ptr(), None) < 0
    assert lib.lr_sample_topk(logits.data_ptr(), 100, noise.data_ptr(), 640, 2, 640, 0.8, 200, None, 0, out.data_ptr(),
                              None) < 0
