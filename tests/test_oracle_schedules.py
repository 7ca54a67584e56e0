"""Pins the block schedules of oracle/ladder_oracle.py (ladder, dense, desync, parallel), the
rank-shard layout and the generation loop through brute-force recurrences, special cases that
collapse to something simpler, and negative controls."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ladder_oracle as O


def tiny(**kw):
    base = dict(block_size=32, vocab_size=96, n_layer=3, n_head=4, n_local_heads=2, dim=32, intermediate_size=48,
                rope_base=10000)
    base.update(kw)
    return O.OracleConfig(**base)


def run(cfg, P, family, idx, pos, B=None, smax=16):
    caches = O.setup_caches(cfg, idx.shape[0] if B is None else B, smax, P["output.weight"].dtype)
    return O.FORWARD[family](cfg, P, caches, idx, pos), caches


def big_params(cfg, family="ladder", seed=0):
    # std 0.5 so that every term matters in fp32 comparisons
    return O.init_params(cfg, family, seed=seed, std=0.5)


IDX = torch.tensor([[3, 17, 60, 5, 9], [8, 8, 1, 0, 95]])
POS = torch.arange(5)


# ------------------------------------------------------------------ ladder (gpt_ladder_TP.py:252-284, 312-358)

def test_ladder_equals_generic_stale_input_recurrence():
    """Module i (attn_0, mlp_0, attn_1, ...) reads the stream WITHOUT the output of module i-1:
    r_i = r_{i-1} + h_{i-2}(...).  Re-derived here with a flat list of 2L modules."""
    cfg = tiny()
    P = big_params(cfg)
    logits, _ = run(cfg, P, "ladder", IDX, POS)

    caches = O.setup_caches(cfg, 2, 16, torch.float32)
    fc, mask = caches.freqs_cis[POS], caches.causal_mask[POS]
    mods = []
    for i in range(cfg.n_layer):
        mods.append(lambda r, i=i: O.attention(cfg, P, i, O.rms_norm(r, P[f"layers.{i}.attention_norm.weight"],
                                                                     cfg.norm_eps), caches, fc, mask, POS))
        mods.append(lambda r, i=i: O.feed_forward(cfg, P, i, O.rms_norm(r, P[f"layers.{i}.ffn_norm.weight"],
                                                                        cfg.norm_eps)))
    r = F.embedding(IDX, P["tok_embeddings.weight"])
    outs = []
    for i, h in enumerate(mods):
        if i >= 2:
            r = r + outs[i - 2]          # the output two modules back has "arrived"
        outs.append(h(r))
    r = r + outs[-2] + outs[-1]
    want = F.linear(O.rms_norm(r, P["norm.weight"], cfg.norm_eps), P["output.weight"])
    assert torch.allclose(logits, want, rtol=1e-5, atol=1e-5)


def test_ladder_single_layer_and_zero_output_projections():
    cfg = tiny(n_layer=1)
    P = big_params(cfg)
    logits, caches = run(cfg, P, "ladder", IDX, POS)
    emb = F.embedding(IDX, P["tok_embeddings.weight"])
    c2 = O.setup_caches(cfg, 2, 16, torch.float32)
    a = O.attention(cfg, P, 0, O.rms_norm(emb, P["layers.0.attention_norm.weight"], cfg.norm_eps), c2,
                    c2.freqs_cis[POS], c2.causal_mask[POS], POS)
    m = O.feed_forward(cfg, P, 0, O.rms_norm(emb, P["layers.0.ffn_norm.weight"], cfg.norm_eps))  # sees emb, not emb+a
    want = F.linear(O.rms_norm(emb + a + m, P["norm.weight"], cfg.norm_eps), P["output.weight"])
    assert torch.allclose(logits, want, rtol=1e-5, atol=1e-5)

    cfg = tiny()
    P = big_params(cfg)
    for i in range(cfg.n_layer):
        P[f"layers.{i}.attention.wo.weight"].zero_()
        P[f"layers.{i}.feed_forward.w2.weight"].zero_()
    logits, _ = run(cfg, P, "ladder", IDX, POS)
    want = F.linear(O.rms_norm(F.embedding(IDX, P["tok_embeddings.weight"]), P["norm.weight"], cfg.norm_eps),
                    P["output.weight"])
    assert torch.allclose(logits, want, atol=1e-6)


def test_ladder_differs_from_dense_negative_control():
    cfg = tiny(n_layer=1)
    P = big_params(cfg)
    a, _ = run(cfg, P, "ladder", IDX, POS)
    b, _ = run(cfg, P, "dense", IDX, POS)
    assert (a - b).abs().max() > 1e-2


# ------------------------------------------------------------------ dense / desync / parallel

def test_dense_is_the_textbook_prenorm_block():
    cfg = tiny(n_layer=2)
    P = big_params(cfg)
    logits, _ = run(cfg, P, "dense", IDX, POS)
    caches = O.setup_caches(cfg, 2, 16, torch.float32)
    x = F.embedding(IDX, P["tok_embeddings.weight"])
    for i in range(2):
        x = x + O.attention(cfg, P, i, O.rms_norm(x, P[f"layers.{i}.attention_norm.weight"], cfg.norm_eps), caches,
                            caches.freqs_cis[POS], caches.causal_mask[POS], POS)
        x = x + O.feed_forward(cfg, P, i, O.rms_norm(x, P[f"layers.{i}.ffn_norm.weight"], cfg.norm_eps))
    want = F.linear(O.rms_norm(x, P["norm.weight"], cfg.norm_eps), P["output.weight"])
    assert torch.equal(logits, want)


@pytest.mark.parametrize("pattern", ["all", "none", "default"])
def test_desync_at_tp1_equals_dense(pattern):
    kw = {}
    if pattern == "all":
        kw["reduce_pattern"] = [{"attention": True, "mlp": True}] * 3
    elif pattern == "none":  # the "upper-bound" configs: never reduce (gpt_desync_TP.py:92-113)
        kw["reduce_pattern"] = [{"attention": False, "mlp": False}] * 3
        kw["force_disable_last_all_reduce"] = True
    cfg = tiny(**kw)
    P = big_params(cfg)
    a, _ = run(cfg, P, "desync", IDX, POS)
    b, _ = run(cfg, P, "dense", IDX, POS)
    assert torch.equal(a, b)  # x / 1 is exact


def test_desync_flags_and_residual_prescale():
    cfg = tiny(n_layer=3, reduce_pattern=[{"attention": False, "mlp": False}] * 3)
    assert [O.desync_flags(cfg, i) for i in range(3)] == [(False, False), (False, False), (False, True)]
    cfg = tiny(n_layer=3, reduce_pattern=[{"attention": True, "mlp": False}] * 3, force_disable_last_all_reduce=True)
    assert [O.desync_flags(cfg, i) for i in range(3)] == [(True, False), (True, False), (True, False)]
    assert O.desync_flags(tiny(n_layer=2), 0) == (False, True)  # default pattern (gpt_desync_TP.py:59-60)

    # with tp = 2 the residual entering a reducing add is divided by 2: check one layer by hand
    cfg = tiny(n_layer=1, n_head=4, n_local_heads=2, tp_world_size=2,
               reduce_pattern=[{"attention": True, "mlp": False}], force_disable_last_all_reduce=True)
    P = big_params(cfg, "desync")
    logits, _ = run(cfg, P, "desync", IDX, POS)
    caches = O.setup_caches(cfg, 2, 16, torch.float32)
    x = F.embedding(IDX, P["tok_embeddings.weight"])
    x = O.attention(cfg, P, 0, O.rms_norm(x, P["layers.0.attention_norm.weight"], cfg.norm_eps), caches,
                    caches.freqs_cis[POS], caches.causal_mask[POS], POS) + x / 2
    x = O.feed_forward(cfg, P, 0, O.rms_norm(x, P["layers.0.ffn_norm.weight"], cfg.norm_eps)) + x
    want = F.linear(O.rms_norm(x, P["norm.weight"], cfg.norm_eps), P["output.weight"])
    assert torch.allclose(logits, want, rtol=1e-5, atol=1e-5)


def test_parallel_equals_attention_plus_mlp_on_the_same_normed_input():
    cfg = tiny(n_layer=2)
    Pl = big_params(cfg, "ladder")
    Pp = {k: v for k, v in Pl.items() if ".layers." not in k and not k.startswith("layers.")}
    for i in range(2):
        p = f"layers.{i}."
        Pp[p + "attention.wqkv1.weight"] = torch.cat([Pl[p + "attention.wqkv.weight"], Pl[p + "feed_forward.w1.weight"]])
        Pp[p + "attention.wo.weight"] = Pl[p + "attention.wo.weight"]
        Pp[p + "attention.w2.weight"] = Pl[p + "feed_forward.w2.weight"]
        Pp[p + "attention_norm.weight"] = Pl[p + "attention_norm.weight"]
    logits, _ = run(cfg, Pp, "parallel", IDX, POS)
    caches = O.setup_caches(cfg, 2, 16, torch.float32)
    x = F.embedding(IDX, Pl["tok_embeddings.weight"])
    for i in range(2):
        n = O.rms_norm(x, Pl[f"layers.{i}.attention_norm.weight"], cfg.norm_eps)
        y = O.attention(cfg, Pl, i, n, caches, caches.freqs_cis[POS], caches.causal_mask[POS], POS)
        x = (O.feed_forward(cfg, Pl, i, n) + y) + x
    want = F.linear(O.rms_norm(x, Pl["norm.weight"], cfg.norm_eps), Pl["output.weight"])
    assert torch.allclose(logits, want, rtol=1e-5, atol=1e-5)
    assert [n for n, _ in O.param_shapes(cfg, "parallel")][1:5] == [
        "layers.0.attention.wqkv1.weight", "layers.0.attention.wo.weight", "layers.0.attention.w2.weight",
        "layers.0.attention_norm.weight"]


# ------------------------------------------------------------------ rank shards (utils.py:142-143, 165-166, 174-176)

def shard_params(cfg_full, P, rank, tp):
    """Slice an un-sharded parameter set into rank `rank` of `tp`: column-parallel wqkv / w1 keep
    rows [q_r; k_r; v_r] / [u_r; g_r], row-parallel wo / w2 keep the matching input columns."""
    hd = cfg_full.head_dim
    hq, hkv, I = cfg_full.n_head // tp, cfg_full.n_local_heads // tp, cfg_full.intermediate_size // tp
    nq, nkv, If = cfg_full.n_head * hd, cfg_full.n_local_heads * hd, cfg_full.intermediate_size
    out = {}
    for k, w in P.items():
        if k.endswith("wqkv.weight"):
            q, kk, v = w.split([nq, nkv, nkv])
            out[k] = torch.cat([q[rank * hq * hd:(rank + 1) * hq * hd], kk[rank * hkv * hd:(rank + 1) * hkv * hd],
                                v[rank * hkv * hd:(rank + 1) * hkv * hd]])
        elif k.endswith("wo.weight"):
            out[k] = w[:, rank * hq * hd:(rank + 1) * hq * hd]
        elif k.endswith("w1.weight"):
            u, g = w.split([If, If])
            out[k] = torch.cat([u[rank * I:(rank + 1) * I], g[rank * I:(rank + 1) * I]])
        elif k.endswith("w2.weight"):
            out[k] = w[:, rank * I:(rank + 1) * I]
        else:
            out[k] = w
    return out


def test_sum_of_rank_partials_equals_unsharded_module():
    """The all-reduce is replaced by 'keep the partial': the partials of all ranks must add up to
    the un-sharded attention / MLP output.  Pins which rows and columns a rank shard holds."""
    tp = 4
    full = tiny(n_layer=1, n_head=8, n_local_heads=4, dim=64, intermediate_size=96)
    P = big_params(full)
    x = torch.randn(2, 5, 64, generator=torch.Generator().manual_seed(3))

    def modules(cfg, params):
        c = O.setup_caches(cfg, 2, 16, torch.float32)
        a = O.attention(cfg, params, 0, x, c, c.freqs_cis[POS], c.causal_mask[POS], POS)
        m = O.feed_forward(cfg, params, 0, x)
        return a.double(), m.double()

    a_full, m_full = modules(full, P)
    shard_cfg = tiny(n_layer=1, n_head=8, n_local_heads=4, dim=64, intermediate_size=96, tp_world_size=tp)
    a_sum = m_sum = 0
    for r in range(tp):
        Pr = shard_params(full, P, r, tp)
        for (name, shape) in O.param_shapes(shard_cfg):
            assert tuple(Pr[name].shape) == shape, name      # the oracle's per-rank shapes are these slices
        a, m = modules(shard_cfg, Pr)
        a_sum, m_sum = a_sum + a, m_sum + m
    assert a_full.abs().max() > 1 and m_full.abs().max() > 1
    assert torch.allclose(a_sum, a_full, rtol=1e-4, atol=1e-4)
    assert torch.allclose(m_sum, m_full, rtol=1e-4, atol=1e-4)


def test_rank_shard_forward_uses_divided_sizes_and_vocab_shard():
    cfg = tiny(n_layer=2, n_head=8, n_local_heads=4, dim=64, intermediate_size=96, tp_world_size=4, vocab_shard=24)
    shapes = dict(O.param_shapes(cfg))
    assert shapes["layers.0.attention.wqkv.weight"] == ((2 + 2 * 1) * 8, 64)
    assert shapes["layers.0.attention.wo.weight"] == (64, 16)
    assert shapes["layers.0.feed_forward.w1.weight"] == (48, 64)
    assert shapes["layers.0.feed_forward.w2.weight"] == (64, 24)
    assert shapes["output.weight"] == (24, 64) and shapes["tok_embeddings.weight"] == (96, 64)
    P = big_params(cfg)
    logits, caches = run(cfg, P, "ladder", IDX, POS)
    assert logits.shape == (2, 5, 24) and caches.k[0].shape == (2, 1, 16, 8)


# ------------------------------------------------------------------ caches and the generation loop

def test_setup_caches_shapes_and_rounding():
    cfg = tiny()
    c = O.setup_caches(cfg, 3, 13, torch.bfloat16)
    assert c.max_seq_length == 16 and c.k[0].shape == (3, 2, 16, 8) and len(c.k) == 3
    assert c.freqs_cis.shape == (32, 4, 2) and c.freqs_cis.dtype == torch.bfloat16
    assert c.causal_mask.shape == (16, 16) and c.causal_mask[3].tolist() == [True] * 4 + [False] * 12


@pytest.mark.parametrize("family", ["ladder", "dense", "desync", "parallel"])
def test_prefill_then_decode_equals_one_longer_prefill(family):
    cfg = tiny()
    P = big_params(cfg, family)
    idx = torch.tensor([[5, 9, 33, 2, 71, 18, 40]])
    full, _ = run(cfg, P, family, idx, torch.arange(7))
    caches = O.setup_caches(cfg, 1, 16, torch.float32)
    fwd = O.FORWARD[family]
    fwd(cfg, P, caches, idx[:, :4], torch.arange(4))
    for t in range(4, 7):
        step = fwd(cfg, P, caches, idx[:, t:t + 1], torch.tensor([t], dtype=torch.int))
        assert torch.allclose(step[:, 0], full[:, t], rtol=1e-4, atol=1e-4)
    # slots beyond the last written position stay zero
    assert caches.k[0][:, :, 7:].abs().sum() == 0 and caches.v[1][:, :, 7:].abs().sum() == 0


def test_generate_loop_lengths_and_teacher_forcing():
    cfg = tiny()
    P = big_params(cfg)
    prompt = torch.tensor([4, 8, 15, 16, 23, 42])
    toks, logits = O.generate(cfg, P, prompt, max_new_tokens=5, batch_size=2)
    assert toks.shape == (2, 5) and toks.dtype == torch.int32 and logits.shape == (5, 2, 96)
    assert torch.equal(toks[0], toks[1])                      # same prompt in every row (benchmark.py:136)
    assert torch.equal(toks, logits.argmax(-1).T.to(torch.int32))
    # replay by hand: prefill + (max_new_tokens - 1) decode steps at positions T, T+1, ...
    caches = O.setup_caches(cfg, 2, 11, torch.float32)
    x = prompt.view(1, -1).repeat(2, 1)
    lg = O.forward_ladder(cfg, P, caches, x, torch.arange(6))
    seq = [lg[:, -1].argmax(-1, keepdim=True)]
    for i in range(4):
        lg = O.forward_ladder(cfg, P, caches, seq[-1], torch.tensor([6 + i]))
        seq.append(lg[:, -1].argmax(-1, keepdim=True))
    assert torch.equal(torch.cat(seq, 1).to(torch.int32), toks)
    # teacher forcing feeds the given tokens but still reports the oracle's own argmax
    forced = torch.full((2, 5), 7)
    t2, l2 = O.generate(cfg, P, prompt, 5, 2, forced=forced)
    assert torch.equal(t2[:, 0], toks[:, 0]) and torch.equal(l2[0], logits[0])
    assert not torch.equal(l2[2], logits[2])


def test_init_params_every_parameter_normal_and_seeded():
    cfg = tiny()
    a = O.init_params(cfg, seed=0, dtype=torch.bfloat16)
    b = O.init_params(cfg, seed=0, dtype=torch.bfloat16)
    c = O.init_params(cfg, seed=1, dtype=torch.bfloat16)
    assert all(torch.equal(a[k], b[k]) for k in a) and not torch.equal(a["norm.weight"], c["norm.weight"])
    # norm gains are N(0, 0.02) too, not ones (benchmark.py:242-243)
    g = torch.cat([v.float().flatten() for k, v in a.items() if "norm" in k])
    assert abs(g.mean()) < 0.01 and 0.01 < g.std() < 0.03
    w = a["tok_embeddings.weight"].float()
    assert abs(w.std() - 0.02) < 0.002
