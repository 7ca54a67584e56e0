"""Committed golden vectors (tests/golden/tiny_*.npz, written by tests/golden/make_golden.py).

CPU: the oracle must still reproduce them (they freeze its rounding points and schedules).
GPU: the HIP models, loaded with the fixture's parameters, must match them to the stated tolerance
     (logits within 2e-2 of the largest logit when teacher-forced on the fixture's tokens; the
     greedy token equal to the fixture's unless the fixture's own margin is within 2 bf16 ulp)."""
import os

import numpy as np
import pytest
import torch

from oracle import ladder_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
FAMILIES = ("ladder", "dense", "desync", "parallel")
CFG = dict(block_size=64, vocab_size=256, n_layer=3, n_head=2, n_local_heads=1, dim=128, intermediate_size=256,
           rope_base=10000)
DESYNC_PATTERN = [{"attention": False, "mlp": True}, {"attention": True, "mlp": False},
                  {"attention": False, "mlp": False}]


def from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def load(family):
    z = np.load(os.path.join(HERE, "golden", f"tiny_{family}.npz"))
    P = {k[len("param:"):]: from_bits(z[k]) for k in z.files if k.startswith("param:")}
    B, T, NEW = (int(v) for v in z["shape"])
    return P, torch.from_numpy(z["prompt"]), torch.from_numpy(z["tokens"]), from_bits(z["logits"]), (B, T, NEW)


def cfg_kw(family):
    kw = dict(CFG)
    if family == "desync":
        kw["reduce_pattern"] = DESYNC_PATTERN
    return kw


@pytest.mark.parametrize("family", FAMILIES)
def test_oracle_reproduces_fixture(family):
    P, prompt, tokens, logits, (B, T, NEW) = load(family)
    cfg = O.OracleConfig(**cfg_kw(family))
    assert sorted(P) == sorted(n for n, _ in O.param_shapes(cfg, family))
    tok, lg = O.generate(cfg, P, prompt, NEW, B, family)
    lg = torch.stack(list(lg)).float()
    # same arithmetic; only the CPU matmul's summation order may differ between machines
    assert ((lg - logits.float()).abs().max() / logits.float().abs().max()).item() <= 1e-2
    assert (tok == tokens).float().mean().item() >= 0.8
    assert torch.equal(tok[0], tok[1]), "identical batch rows must decode identically"


def test_fixtures_tell_the_schedules_apart():
    lad, den, des, par = (load(f)[3].float() for f in FAMILIES)
    assert (lad - den).abs().max() > 0.1 * den.abs().max()      # ladder is not dense
    assert (par - den).abs().max() > 0.1 * den.abs().max()      # parallel is not dense
    assert torch.equal(des, den) or (des - den).abs().max() <= 1e-2 * den.abs().max()   # one rank: desync == dense


@pytest.mark.gpu
@pytest.mark.parametrize("family,fused", [("ladder", True)] + [(f, False) for f in FAMILIES])
def test_hip_matches_fixture(family, fused):
    """fused: the one-kernel decode step (it exists for the ladder schedule only)."""
    import benchmark as bm
    from gpt_fast.config import ModelArgs

    P, prompt, tokens, logits, (B, T, NEW) = load(family)
    cls = {"ladder": bm.GPTLadder, "dense": bm.GPTDense, "desync": bm.GPTDesync, "parallel": bm.GPTParallel}[family]
    with torch.device("meta"):
        model = cls(ModelArgs(**cfg_kw(family)))
    model = model.to(dtype=torch.bfloat16).to_empty(device="cuda").eval()
    missing, unexpected = model.load_state_dict({k: v.cuda() for k, v in P.items()}, strict=False)
    assert not unexpected and all("kv_cache" in m or "freqs" in m or "mask" in m for m in missing), (missing, unexpected)
    if family == "ladder":
        model.use_fused_step = fused
    logits, tokens, prompt = logits.cuda().float(), tokens.cuda(), prompt.cuda()
    scale = logits.abs().max()
    with torch.no_grad():
        model.setup_caches(B, T + NEW)
        out = model(prompt.view(1, -1).repeat(B, 1), torch.arange(T, device="cuda"))
        pos = torch.tensor([T], dtype=torch.int32, device="cuda")
        for i in range(NEW):
            got = out[:, -1].float()
            assert ((got - logits[i]).abs().max() / scale).item() <= 2e-2, (family, i)
            tok = model.greedy_next(out).view(-1)
            top = logits[i].max(-1).values
            at = logits[i].gather(-1, tok.long().view(-1, 1)).squeeze(-1)
            ulp = top.abs().log2().floor().exp2() * 2.0 ** -7
            assert bool(((tok == tokens[:, i]) | (top - at <= 2 * ulp)).all()), (family, i, tok, tokens[:, i])
            if i + 1 < NEW:
                out = model(tokens[:, i:i + 1].contiguous(), pos)
                pos += 1
    if family == "ladder" and fused:
        fs = model._fused_step(B)
        assert fs is not None and not fs.failed()
