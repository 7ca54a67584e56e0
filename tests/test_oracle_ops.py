"""Pins each op of oracle/ladder_oracle.py against something that is NOT the oracle's own
formula: a closed form evaluated in float64 with integer-arithmetic bf16 rounding, a library
routine, brute-force loops on tiny inputs, or an invariant chosen so that a plausible mistake
(dropped term, wrong sign or index, transposed operand, wrong rounding point) fails.

The reference (mayank31398/ladder-residual-inference) holds no tests, fixtures or golden
vectors, so these checks are what fixes the oracle."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import bf16_round_np
from oracle import ladder_oracle as O


def _rng(seed=0):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


# ------------------------------------------------------------------ RMSNorm (utils.py:68-74)

def test_rmsnorm_fp64_closed_form_with_two_roundings():
    g = _rng(1)
    x = (torch.randn(5, 96, generator=g) * 3).to(torch.bfloat16)
    w = (torch.randn(96, generator=g) * 0.02).to(torch.bfloat16)
    got = O.rms_norm(x, w, 1e-5).float().numpy()
    x64 = x.double().numpy()
    w64 = w.double().numpy()
    n = bf16_round_np(x64 / np.sqrt((x64 * x64).mean(-1, keepdims=True) + 1e-5))  # rounding point 1
    want = bf16_round_np(n.astype(np.float64) * w64)                               # rounding point 2
    # fp32-vs-fp64 rsqrt may move a value sitting on a rounding boundary: allow a few 1-ulp cases
    bad = got != want
    assert bad.mean() < 0.01
    assert np.all(np.abs(got - want)[bad] <= np.abs(want[bad]) * 2.0 ** -7)


def test_rmsnorm_rounding_order_is_distinguishable():
    """Negative control: gain applied BEFORE the rounding (what F.rms_norm does) differs."""
    g = _rng(2)
    x = torch.randn(64, 512, generator=g).to(torch.bfloat16)
    w = (torch.randn(512, generator=g) * 0.02).to(torch.bfloat16)
    ours = O.rms_norm(x, w, 1e-5)
    xf = x.float()
    fused = (xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + 1e-5) * w.float()).to(torch.bfloat16)
    assert (ours != fused).float().mean() > 0.01


def test_rmsnorm_invariants_fp32():
    g = _rng(3)
    x = torch.randn(4, 256, generator=g)
    w = torch.randn(256, generator=g)
    y = O.rms_norm(x, w, 0.0)
    # unit gain -> unit RMS; scale invariance in x; linearity in the gain
    assert torch.allclose(O.rms_norm(x, torch.ones(256), 0.0).pow(2).mean(-1), torch.ones(4), atol=1e-5)
    assert torch.allclose(O.rms_norm(7.5 * x, w, 0.0), y, atol=1e-5)
    assert torch.allclose(O.rms_norm(x, 3 * w, 0.0), 3 * y, atol=1e-5)
    # eps enters inside the square root, added to the MEAN (not the sum) of squares
    x1 = torch.full((1, 16), 2.0)
    assert torch.allclose(O.rms_norm(x1, torch.ones(16), 5.0), x1 / math.sqrt(4.0 + 5.0))


# ------------------------------------------------------------------ RoPE table (utils.py:103-117)

def test_rope_table_closed_form():
    hd, base, n = 128, 500000.0, 300
    tab = O.rope_table(n, hd, base, torch.float32)
    assert tab.shape == (n, hd // 2, 2)
    j = np.arange(hd // 2, dtype=np.float64)
    f64 = base ** (-2 * j / hd)
    ang = np.arange(n, dtype=np.float64)[:, None] * f64[None, :]
    f_got = np.arctan2(tab[1, :, 1].double().numpy(), tab[1, :, 0].double().numpy())  # angle at t=1
    assert np.allclose(f_got, f64, rtol=2e-6)
    # the reference forms frequency and angle in fp32: the error allowed grows with the angle
    tol = 4e-7 * (1.0 + ang)
    assert np.all(np.abs(tab[..., 0].double().numpy() - np.cos(ang)) <= tol)
    assert np.all(np.abs(tab[..., 1].double().numpy() - np.sin(ang)) <= tol)
    # (cos, sin) == real/imag of torch.polar(1, angle), the reference's formulation
    fr = 1.0 / (base ** (torch.arange(0, hd, 2)[: hd // 2].float() / hd))
    pol = torch.polar(torch.ones(n, hd // 2), torch.outer(torch.arange(n), fr))
    assert np.abs((tab[..., 0] - pol.real).numpy()).max() < 2e-7
    assert np.abs((tab[..., 1] - pol.imag).numpy()).max() < 2e-7


def test_rope_table_is_rounded_to_model_dtype():
    a = O.rope_table(64, 64, 10000, torch.bfloat16)
    b = O.rope_table(64, 64, 10000, torch.float32)
    assert a.dtype == torch.bfloat16
    assert np.array_equal(a.float().numpy(), bf16_round_np(b.numpy()))
    assert torch.all(a[0, :, 0] == 1) and torch.all(a[0, :, 1] == 0)


LLAMA31 = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)


def test_rope_scaling_piecewise_closed_form():
    hd, base = 128, 500000.0
    f = 1.0 / (base ** (torch.arange(0, hd, 2).float() / hd))
    got = O.rope_scaled_freqs(f, LLAMA31).double().numpy()
    f64 = f.double().numpy()
    wl = 2 * math.pi / f64
    want = np.where(wl < 8192 / 4.0, f64, np.where(wl > 8192 / 1.0, f64 / 8.0, 0.0))
    mid = (wl >= 8192 / 4.0) & (wl <= 8192 / 1.0)
    smooth = (8192 / wl - 1.0) / (4.0 - 1.0)
    want = np.where(mid, (1 - smooth) * f64 / 8.0 + smooth * f64, want)
    assert mid.sum() > 0 and (wl < 2048).sum() > 0 and (wl > 8192).sum() > 0  # all three bands hit
    assert np.allclose(got, want, rtol=3e-6)


def test_rope_scaling_matches_transformers_llama3():
    tr = pytest.importorskip("transformers")
    try:
        from transformers.modeling_rope_utils import _compute_llama3_parameters
        cfg = tr.LlamaConfig(hidden_size=16384, num_attention_heads=128, max_position_embeddings=131072,
                             rope_parameters=dict(rope_type="llama3", rope_theta=500000.0, **LLAMA31))
        inv, _ = _compute_llama3_parameters(cfg, device="cpu")
    except Exception as e:  # API drift of an independent library is not a failure of the oracle
        pytest.skip(f"transformers llama3 helper not callable here: {e}")
    f = 1.0 / (500000.0 ** (torch.arange(0, 128, 2).float() / 128))
    assert torch.allclose(O.rope_scaled_freqs(f, LLAMA31), inv.float(), rtol=3e-6, atol=0)


# ------------------------------------------------------------------ RoPE apply (utils.py:120-132)

def test_rope_equals_complex_multiplication():
    g = _rng(4)
    B, S, H, hd = 2, 7, 3, 64
    x = torch.randn(B, S, H, hd, generator=g)
    tab = O.rope_table(32, hd, 10000, torch.float32)[5:5 + S]
    got = O.apply_rope(x, tab)
    xc = torch.view_as_complex(x.double().reshape(B, S, H, hd // 2, 2))
    rot = torch.view_as_complex(tab.double().contiguous()).view(1, S, 1, hd // 2)
    want = torch.view_as_real(xc * rot).flatten(3)
    assert torch.allclose(got.double(), want, atol=1e-6)


def test_rope_invariants_and_half_split_form():
    g = _rng(5)
    B, S, H, hd = 1, 6, 2, 32
    x = torch.randn(B, S, H, hd, generator=g)
    tab = O.rope_table(S, hd, 10000, torch.float32)
    y = O.apply_rope(x, tab)
    assert torch.equal(y[:, 0], x[:, 0])                                           # position 0: identity
    pairs = lambda t: t.reshape(B, S, H, hd // 2, 2).pow(2).sum(-1)
    assert torch.allclose(pairs(y), pairs(x), atol=1e-5)                           # per-pair norm kept
    # equals the "rotate_half" form after the even/odd -> half-split permutation
    perm = torch.cat([torch.arange(0, hd, 2), torch.arange(1, hd, 2)])
    xh = x[..., perm]
    cos = torch.cat([tab[..., 0], tab[..., 0]], -1).view(1, S, 1, hd)
    sin = torch.cat([tab[..., 1], tab[..., 1]], -1).view(1, S, 1, hd)
    rot_half = torch.cat([-xh[..., hd // 2:], xh[..., : hd // 2]], -1)
    assert torch.allclose(y[..., perm], xh * cos + rot_half * sin, atol=1e-6)


def test_rope_bf16_table_promoted_and_single_rounding():
    g = _rng(6)
    x = torch.randn(1, 4, 2, 64, generator=g).to(torch.bfloat16)
    tab = O.rope_table(16, 64, 500000, torch.bfloat16)[3:7]
    got = O.apply_rope(x, tab).float().numpy()
    x64 = x.double().numpy().reshape(1, 4, 2, 32, 2)
    c = tab[..., 0].double().numpy().reshape(1, 4, 1, 32)
    s = tab[..., 1].double().numpy().reshape(1, 4, 1, 32)
    want = np.stack([x64[..., 0] * c - x64[..., 1] * s, x64[..., 1] * c + x64[..., 0] * s], -1).reshape(1, 4, 2, 64)
    want = bf16_round_np(want)
    bad = got != want
    assert bad.mean() < 0.01 and np.all(np.abs(got - want)[bad] <= np.abs(want[bad]) * 2.0 ** -7)


# ------------------------------------------------------------------ KV cache (utils.py:50-59)

def test_kv_update_writes_only_the_addressed_slots():
    kc = torch.zeros(2, 2, 16, 8)
    vc = torch.zeros(2, 2, 16, 8)
    k = torch.arange(2 * 2 * 3 * 8, dtype=torch.float32).view(2, 2, 3, 8) + 1
    O.kv_update(kc, vc, torch.tensor([4, 5, 9]), k, -k)
    assert torch.equal(kc[:, :, [4, 5, 9]], k) and torch.equal(vc[:, :, [4, 5, 9]], -k)
    rest = [i for i in range(16) if i not in (4, 5, 9)]
    assert kc[:, :, rest].abs().sum() == 0 and vc[:, :, rest].abs().sum() == 0


# ------------------------------------------------------------------ attention (utils.py:252-255)

def _brute_attention(q, k, v, mask):
    """float64 loops.  q [B,Hq,S,hd], k/v [B,Hkv,Smax,hd], mask [S,Smax]."""
    B, Hq, S, hd = q.shape
    G = Hq // k.shape[1]
    out = np.zeros((B, Hq, S, hd))
    for b in range(B):
        for h in range(Hq):
            for s in range(S):
                sc = np.array([np.dot(q[b, h, s], k[b, h // G, j]) / math.sqrt(hd) if mask[s, j] else -np.inf
                               for j in range(k.shape[2])])
                p = np.exp(sc - sc.max())
                p /= p.sum()
                out[b, h, s] = (p[:, None] * v[b, h // G]).sum(0)
    return out


def test_sdpa_math_brute_force_gqa_and_mask():
    g = _rng(7)
    B, Hq, Hkv, S, Smax, hd = 2, 4, 2, 3, 8, 16
    q = torch.randn(B, Hq, S, hd, generator=g)
    k = torch.randn(B, Hkv, Smax, hd, generator=g)
    v = torch.randn(B, Hkv, Smax, hd, generator=g)
    pos = torch.tensor([2, 3, 4])
    mask = torch.tril(torch.ones(Smax, Smax, dtype=torch.bool))[pos]
    got = O.sdpa_math(q, k, v, mask).double().numpy()
    want = _brute_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), mask.numpy())
    assert np.abs(got - want).max() < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sdpa_math_matches_library_routine(dtype):
    g = _rng(8)
    B, Hq, Hkv, S, Smax, hd = 2, 8, 2, 5, 24, 64
    q = torch.randn(B, Hq, S, hd, generator=g).to(dtype)
    k = torch.randn(B, Hkv, Smax, hd, generator=g).to(dtype)
    v = torch.randn(B, Hkv, Smax, hd, generator=g).to(dtype)
    pos = torch.arange(10, 10 + S)
    mask = torch.tril(torch.ones(Smax, Smax, dtype=torch.bool))[pos]
    from torch.nn.attention import SDPBackend, sdpa_kernel

    with sdpa_kernel(SDPBackend.MATH):  # the reference forces the math backend (benchmark.py:107,142)
        want = F.scaled_dot_product_attention(q, k.repeat_interleave(Hq // Hkv, 1),
                                              v.repeat_interleave(Hq // Hkv, 1),
                                              attn_mask=mask[None, None], dropout_p=0.0)
    got = O.sdpa_math(q, k, v, mask)
    if dtype == torch.float32:
        assert torch.allclose(got, want, atol=2e-6)
    else:  # fp32 inside, one rounding at the end: at most rare 1-ulp boundary cases
        diff = (got.float() - want.float()).abs()
        assert (diff > 0).float().mean() < 0.02 and torch.all(diff <= want.float().abs() * 2.0 ** -7 + 1e-30)


def test_sdpa_invariants():
    g = _rng(9)
    B, Hq, Hkv, hd = 1, 4, 1, 32
    q = torch.randn(B, Hq, 1, hd, generator=g)
    k = torch.randn(B, Hkv, 16, hd, generator=g)
    v = torch.randn(B, Hkv, 16, hd, generator=g)
    tril = torch.tril(torch.ones(16, 16, dtype=torch.bool))
    # pos = 0: a single visible key -> output is v[0] for every q head
    y0 = O.sdpa_math(q, k, v, tril[[0]])
    assert torch.allclose(y0, v[:, :, 0:1].expand(B, Hq, 1, hd), atol=1e-6)
    # masked slots contribute nothing: the result does not depend on Smax or on garbage beyond pos
    y5 = O.sdpa_math(q, k, v, tril[[5]])
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 6:] = 1e3
    v2[:, :, 6:] = -1e3
    assert torch.equal(O.sdpa_math(q, k2, v2, tril[[5]]), y5)
    assert torch.allclose(O.sdpa_math(q, k[:, :, :8], v[:, :, :8], tril[:8, :8][[5]]), y5, atol=1e-6)


# ------------------------------------------------------------------ SwiGLU / linears (utils.py:145-149)

def test_feed_forward_chunk_order_and_rounding():
    cfg = O.OracleConfig(dim=32, n_head=2, n_layer=1, intermediate_size=48, vocab_size=64)
    g = _rng(10)
    w1 = torch.randn(96, 32, generator=g).to(torch.bfloat16)
    w2 = torch.randn(32, 48, generator=g).to(torch.bfloat16)
    x = torch.randn(1, 3, 32, generator=g).to(torch.bfloat16)
    P = {"layers.0.feed_forward.w1.weight": w1, "layers.0.feed_forward.w2.weight": w2}
    got = O.feed_forward(cfg, P, 0, x).float().numpy()
    h = bf16_round_np(x.double().numpy() @ w1.double().numpy().T)            # [out, in] layout
    u, gt = h[..., :48].astype(np.float64), h[..., 48:].astype(np.float64)    # FIRST half is "up"
    act = bf16_round_np(gt / (1 + np.exp(-gt)))                               # silu rounded ...
    prod = bf16_round_np(act.astype(np.float64) * u)                          # ... then the product
    want = bf16_round_np(prod.astype(np.float64) @ w2.double().numpy().T)
    bad = got != want
    assert bad.mean() < 0.05 and np.all(np.abs(got - want)[bad] <= np.abs(want[bad]) * 2.0 ** -7)
    # negative control: swapping the halves changes the answer
    swapped = torch.cat([w1[48:], w1[:48]])
    P2 = dict(P, **{"layers.0.feed_forward.w1.weight": swapped})
    assert not torch.equal(O.feed_forward(cfg, P2, 0, x), O.feed_forward(cfg, P, 0, x))


def test_attention_wqkv_row_order_and_layouts():
    """wqkv rows [q; k; v], heads contiguous in hd, cache BHSD: check against float64 loops."""
    cfg = O.OracleConfig(dim=32, n_head=4, n_local_heads=2, n_layer=1, intermediate_size=32, vocab_size=16,
                         block_size=16)
    g = _rng(11)
    hd = 8
    wqkv = torch.randn((4 + 4) * hd, 32, generator=g) * 0.3
    wo = torch.randn(32, 32, generator=g) * 0.3
    P = {"layers.0.attention.wqkv.weight": wqkv, "layers.0.attention.wo.weight": wo}
    caches = O.setup_caches(cfg, 1, 8, torch.float32)
    x = torch.randn(1, 3, 32, generator=g)
    pos = torch.arange(3)
    got = O.attention(cfg, P, 0, x, caches, caches.freqs_cis[pos], caches.causal_mask[pos], pos)

    X = x[0].double().numpy()
    W = wqkv.double().numpy()
    tab = caches.freqs_cis.double().numpy()

    def rope(vec, t):  # vec [hd]
        o = vec.copy()
        for j in range(hd // 2):
            c, s = tab[t, j]
            o[2 * j] = vec[2 * j] * c - vec[2 * j + 1] * s
            o[2 * j + 1] = vec[2 * j + 1] * c + vec[2 * j] * s
        return o

    Q = np.zeros((4, 3, hd)); K = np.zeros((2, 3, hd)); V = np.zeros((2, 3, hd))
    for t in range(3):
        row = W @ X[t]
        for h in range(4):
            Q[h, t] = rope(row[h * hd:(h + 1) * hd], t)
        for h in range(2):
            K[h, t] = rope(row[32 + h * hd: 32 + (h + 1) * hd], t)
            V[h, t] = row[48 + h * hd: 48 + (h + 1) * hd]
    y = _brute_attention(Q[None], K[None], V[None], np.tril(np.ones((3, 3), dtype=bool)))[0]  # [4,3,hd]
    y = y.transpose(1, 0, 2).reshape(3, 32)                                   # [S, Hq*hd]
    want = y @ wo.double().numpy().T
    assert np.abs(got[0].double().numpy() - want).max() < 1e-5
    # the cache holds the ROTATED k and the raw v at the written slots, zeros elsewhere
    assert np.abs(caches.k[0][0, :, :3].double().numpy() - K).max() < 1e-6
    assert np.abs(caches.v[0][0, :, :3].double().numpy() - V).max() < 1e-6
    assert caches.k[0][0, :, 3:].abs().sum() == 0


# ------------------------------------------------------------------ greedy (replaces benchmark.py:73-77)

def test_greedy_first_maximum_on_ties_int32():
    lg = torch.zeros(2, 3, 10)
    lg[0, -1, [4, 7]] = 1.0
    lg[1, -1, [9, 2]] = 3.0
    lg[:, 0, 0] = 100.0  # only the LAST position counts
    t = O.greedy(lg)
    assert t.dtype == torch.int32 and t.shape == (2, 1) and t.flatten().tolist() == [4, 2]
    assert O.greedy(lg.to(torch.bfloat16)).flatten().tolist() == [4, 2]


# ------------------------------------------------------------------------------------ weight-only fp8

def test_fp8_quantiser_closed_forms():
    """quantize_fp8_rowwise / linear_fp8 (the weight-only scheme behind gpt_ladder_TP.py:233-237) against what
    the definition fixes: the row maximum lands on +-448, every element is within half an e4m3 step of the
    scaled weight, a row of zeros stays zero, and the product equals the fp64 product of the de-quantised
    matrix up to the two stated bf16 roundings."""
    g = torch.Generator().manual_seed(0)
    w = torch.randn(33, 64, generator=g) * 0.02
    w[5] = 0.0
    w[7, 3] = 0.5        # a row dominated by one element: the rest falls into the denormal range of e4m3
    q, s = O.quantize_fp8_rowwise(w)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.bfloat16 and s.shape == (33,)
    qf, sf = q.float(), s.float()
    amax = w.abs().amax(1)
    live = amax > 0
    assert torch.equal(qf.abs().amax(1)[live], torch.full((32,), 448.0))
    assert ((sf[live] - amax[live] / 448).abs() <= 2.0 ** -8 * sf[live]).all() and sf[5] == 1.0 and (qf[5] == 0).all()
    # e4m3: 3 mantissa bits -> relative half-step 2^-4 for normal values, absolute half-step 2^-10 below 2^-6
    target = w / sf[:, None]
    err = (qf - target.clamp(-448, 448)).abs()
    assert (err <= torch.maximum(target.abs() * 2.0 ** -4, torch.tensor(2.0 ** -10))).all()
    # a wrong-way division (w * scale) or a dropped clamp would break the lines above; now the product
    x = (torch.randn(5, 64, generator=g)).to(torch.bfloat16)
    y = O.linear_fp8(x, q, s)
    exact = (x.double() @ qf.double().T) * sf.double()
    assert y.dtype == torch.bfloat16
    assert ((y.double() - exact).abs() <= 2.0 ** -7 * exact.abs() + 1e-30).all()
    assert (y[:, 5] == 0).all()
    # and it is NOT the plain linear on the original weights (negative control), though close to it
    plain = torch.nn.functional.linear(x.float(), w)
    assert 1e-3 < ((y.float() - plain).abs().max() / plain.abs().max()).item() < 0.2


def test_fp8_parameter_dict_and_dispatch():
    cfg = O.OracleConfig(block_size=16, vocab_size=64, n_layer=1, n_head=2, dim=32, intermediate_size=48)
    P = O.init_params(cfg, seed=0, dtype=torch.bfloat16, std=0.1)
    Q = O.quantize_params_fp8(P)
    assert Q["tok_embeddings.weight"] is P["tok_embeddings.weight"] and Q["norm.weight"] is P["norm.weight"]
    for n in ("layers.0.attention.wqkv", "layers.0.attention.wo", "layers.0.feed_forward.w1", "layers.0.feed_forward.w2",
              "output"):
        assert Q[n + ".weight"].dtype == torch.float8_e4m3fn and Q[n + ".scales"].shape == (P[n + ".weight"].shape[0],)
    x = torch.randn(3, 32).to(torch.bfloat16)
    assert torch.equal(O.linear(Q, "output.weight", x), O.linear_fp8(x, Q["output.weight"], Q["output.scales"]))
    assert torch.equal(O.linear(P, "output.weight", x), torch.nn.functional.linear(x, P["output.weight"]))
    # the quantised model's logits stay close to the unquantised ones (the scheme is a small perturbation)
    idx = torch.randint(0, 64, (1, 5))
    lp = O.forward_ladder(cfg, P, O.setup_caches(cfg, 1, 16, torch.bfloat16), idx, torch.arange(5)).float()
    lq = O.forward_ladder(cfg, Q, O.setup_caches(cfg, 1, 16, torch.bfloat16), idx, torch.arange(5)).float()
    assert 0 < ((lp - lq).abs().max() / lp.abs().max()).item() < 0.25
