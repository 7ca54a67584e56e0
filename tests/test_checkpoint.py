"""Checkpoint loading (gpt_fast/checkpoint.py): name conversion from Hugging Face Llama-Ladder
checkpoints, per-rank slicing of un-sharded checkpoints, the partial-ladder (`ladder_layers`) wiring.

What pins what:
  * conversion + RoPE row re-ordering + [up; gate] order + partial-ladder schedule: the oracle on the
    converted state dict must reproduce, in fp64, a direct restatement of the HF forward pass in the
    HF names and RoPE layout (tests/hf_ladder_restatement.py) -- for all-ladder, last-n-ladder, a
    ladder block in the middle and no ladder at all;
  * slicing: the sum over ranks of every row-parallel partial output equals the un-sharded module
    output, and the vocab shards concatenate to the full logits (fp64);
  * the loader: parameters of a rank's module equal the slices, dtype cast, strictness.
GPU: a synthetic HF checkpoint on disk -> load_checkpoint -> the HIP model's logits against the oracle."""
import os

import pytest
import torch
import torch.nn.functional as F

from hf_ladder_restatement import hf_ladder_forward, random_hf_state_dict
from oracle import ladder_oracle as O

SHAPE = dict(n_layer=4, n_head=8, n_kv=4, dim=64, ffn=96, vocab=52)


def oracle_logits(P, idx, ladder_layers, tp=1, dtype=torch.float64, vocab_shard=None):
    cfg = O.OracleConfig(block_size=32, vocab_size=SHAPE["vocab"], n_layer=SHAPE["n_layer"], n_head=SHAPE["n_head"],
                         n_local_heads=SHAPE["n_kv"], dim=SHAPE["dim"], intermediate_size=SHAPE["ffn"], rope_base=10000,
                         norm_eps=1e-5, ladder_layers=ladder_layers, tp_world_size=tp, vocab_shard=vocab_shard)
    caches = O.setup_caches(cfg, idx.shape[0], 32, dtype)
    caches.freqs_cis = O.rope_table(32, cfg.head_dim, 10000, dtype)
    return O.forward_ladder(cfg, P, caches, idx, torch.arange(idx.shape[1]))


@pytest.mark.parametrize("ladder_layers", [None, [2, 3], [1, 2], []])
def test_converted_checkpoint_reproduces_the_hf_forward(ladder_layers):
    from gpt_fast.checkpoint import convert_hf_state_dict, is_hf_state_dict

    hf = random_hf_state_dict(**SHAPE)
    assert is_hf_state_dict(hf)
    P = convert_hf_state_dict(hf, SHAPE["n_head"], SHAPE["n_kv"])
    assert not is_hf_state_dict(P)
    idx = torch.randint(0, SHAPE["vocab"], (2, 9), generator=torch.Generator().manual_seed(1))
    want = hf_ladder_forward(hf, idx, SHAPE["n_layer"], SHAPE["n_head"], SHAPE["n_kv"], 10000.0, 1e-5,
                             list(range(SHAPE["n_layer"])) if ladder_layers is None else ladder_layers)
    got = oracle_logits(P, idx, ladder_layers)
    # (the oracle normalises, rotates and attends in fp32 whatever the parameter dtype: agreement to fp32 rounding)
    assert (got - want).abs().max().item() <= 3e-6 * want.abs().max().item()
    # negative controls: without the row re-ordering, or with up and gate swapped, the logits are different
    bad = dict(P)
    bad["layers.0.attention.wqkv.weight"] = torch.cat([hf["model.layers.0.self_attn.q_proj.weight"],
                                                       hf["model.layers.0.self_attn.k_proj.weight"],
                                                       hf["model.layers.0.self_attn.v_proj.weight"]])
    assert (oracle_logits(bad, idx, ladder_layers) - want).abs().max().item() > 1e-3 * want.abs().max().item()
    bad = dict(P)
    u, g = P["layers.1.feed_forward.w1.weight"].chunk(2)
    bad["layers.1.feed_forward.w1.weight"] = torch.cat([g, u])
    assert (oracle_logits(bad, idx, ladder_layers) - want).abs().max().item() > 1e-3 * want.abs().max().item()
    if ladder_layers:   # and the partial-ladder wiring matters
        other = None if ladder_layers != [1, 2] else [2, 3]
        assert (oracle_logits(P, idx, other) - want).abs().max().item() > 1e-3 * want.abs().max().item()


@pytest.mark.parametrize("tp", [2, 4])
@pytest.mark.parametrize("separate_qkv", [False, True])
def test_rank_slices_sum_to_the_unsharded_result(tp, separate_qkv):
    from gpt_fast.checkpoint import convert_hf_state_dict, shard_state_dict

    P = convert_hf_state_dict(random_hf_state_dict(**SHAPE, seed=3), SHAPE["n_head"], SHAPE["n_kv"])
    hd = SHAPE["dim"] // SHAPE["n_head"]
    src = dict(P)
    if separate_qkv:   # the wq / wk / wv form of utils.py:178-185
        for i in range(SHAPE["n_layer"]):
            q, k, v = src.pop(f"layers.{i}.attention.wqkv.weight").split([SHAPE["n_head"] * hd, SHAPE["n_kv"] * hd,
                                                                           SHAPE["n_kv"] * hd])
            src.update({f"layers.{i}.attention.wq.weight": q, f"layers.{i}.attention.wk.weight": k,
                        f"layers.{i}.attention.wv.weight": v})
    shards = [shard_state_dict(src, SHAPE["n_head"], SHAPE["n_kv"], hd, tp, r, shard_vocab=True) for r in range(tp)]
    kw = dict(block_size=32, vocab_size=SHAPE["vocab"], n_layer=SHAPE["n_layer"], n_head=SHAPE["n_head"],
              n_local_heads=SHAPE["n_kv"], dim=SHAPE["dim"], intermediate_size=SHAPE["ffn"], rope_base=10000)
    full, part = O.OracleConfig(**kw), O.OracleConfig(**kw, tp_world_size=tp, vocab_shard=SHAPE["vocab"] // tp)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 7, SHAPE["dim"], generator=g, dtype=torch.float64)
    pos = torch.arange(7)

    def attn(cfg, params):
        c = O.setup_caches(cfg, 2, 32, torch.float64)
        c.freqs_cis = O.rope_table(32, cfg.head_dim, 10000, torch.float64)
        return O.attention(cfg, params, 2, x, c, c.freqs_cis[pos], c.causal_mask[pos], pos)

    want_a, want_m = attn(full, P), O.feed_forward(full, P, 2, x)
    got_a = sum(attn(part, s) for s in shards)
    got_m = sum(O.feed_forward(part, s, 2, x) for s in shards)
    assert (got_a - want_a).abs().max() <= 3e-6 * want_a.abs().max()
    assert (got_m - want_m).abs().max() <= 1e-10 * want_m.abs().max()
    logits = torch.cat([F.linear(x, s["output.weight"]) for s in shards], dim=-1)
    assert torch.equal(logits, F.linear(x, P["output.weight"]))
    # replicated tensors are the same object on every rank; shapes are the reference's per-rank shapes
    assert all(s["tok_embeddings.weight"] is P["tok_embeddings.weight"] for s in shards)
    assert dict((n, tuple(t.shape)) for n, t in shards[1].items()) == \
        dict((n, tuple(sh)) for n, sh in O.param_shapes(part, "ladder"))
    # one rank alone is NOT the answer (negative control)
    assert (attn(part, shards[0]) - want_a).abs().max() > 1e-3 * want_a.abs().max()


def test_model_args_from_the_reference_hf_configs():
    """The fields of hf_modeling_utils/configs/Llama-3.1-8B-Instruct-Ladder-last16L.json."""
    from gpt_fast.checkpoint import model_args_from_hf_config
    from gpt_fast.config import ModelArgs

    hf = {"hidden_size": 4096, "intermediate_size": 14336, "max_position_embeddings": 131072, "num_attention_heads": 32,
          "num_hidden_layers": 32, "num_key_value_heads": 8, "rms_norm_eps": 1e-05, "rope_theta": 500000.0,
          "rope_scaling": {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                           "original_max_position_embeddings": 8192, "rope_type": "llama3"},
          "vocab_size": 128256, "ladder_layers": 16}
    a = ModelArgs(**model_args_from_hf_config(hf, tp_world_size=8, tp_rank=3))
    assert (a.dim, a.n_layer, a.n_head, a.n_local_heads, a.intermediate_size, a.vocab_size, a.head_dim) == \
        (4096, 32, 32, 8, 14336, 128256, 128)
    assert a.ladder_layers == list(range(16, 32)) and a.rope_scaling["factor"] == 8.0 and a.rope_base == 500000.0
    assert not a.is_ladder_layer(15) and a.is_ladder_layer(16) and (a.n_head_local, a.ffn_local) == (4, 1792)
    assert ModelArgs(**model_args_from_hf_config(dict(hf, ladder_layers=32))).ladder_layers is None   # all layers
    # no field at all (a plain Llama config.json) or null: NO ladder layer, every block dense
    # (configuration_llama_ladder.py:38-39) -- not ModelArgs' own default of "all layers"
    plain = {k: v for k, v in hf.items() if k != "ladder_layers"}
    for cfg in (plain, dict(hf, ladder_layers=None)):
        a0 = ModelArgs(**model_args_from_hf_config(cfg))
        assert a0.ladder_layers == [] and not any(a0.is_ladder_layer(i) for i in range(a0.n_layer))
    with pytest.raises(ValueError):
        model_args_from_hf_config(dict(hf, ladder_layers="16"))
    with pytest.raises(ValueError):
        model_args_from_hf_config(dict(hf, rope_scaling={"rope_type": "yarn", "factor": 2.0}))


def test_load_checkpoint_fills_one_rank_and_is_strict(tmp_path):
    import benchmark as bm
    from gpt_fast.checkpoint import convert_hf_state_dict, load_checkpoint, shard_state_dict
    from gpt_fast.config import ModelArgs
    from safetensors.torch import save_file

    hf = random_hf_state_dict(**SHAPE, seed=7, dtype=torch.float32)
    kw = dict(block_size=32, vocab_size=SHAPE["vocab"], n_layer=SHAPE["n_layer"], n_head=SHAPE["n_head"],
              n_local_heads=SHAPE["n_kv"], dim=SHAPE["dim"], intermediate_size=SHAPE["ffn"], tp_world_size=2, tp_rank=1,
              shard_vocab=True, ladder_layers=[2, 3])
    model = bm.GPTLadder(ModelArgs(**kw)).to(torch.bfloat16)
    path = str(tmp_path / "model.safetensors")
    save_file(hf, path)
    loaded = load_checkpoint(model, path)
    want = shard_state_dict(convert_hf_state_dict(hf, SHAPE["n_head"], SHAPE["n_kv"]), SHAPE["n_head"], SHAPE["n_kv"], 8, 2, 1,
                            shard_vocab=True)
    assert sorted(loaded) == sorted(want)
    for n, p in model.named_parameters():
        assert p.dtype == torch.bfloat16 and torch.equal(p, want[n].to(torch.bfloat16)), n
    # a torch file of gpt_fast names loads the same way; a directory of shards too
    torch.save(convert_hf_state_dict(hf, SHAPE["n_head"], SHAPE["n_kv"]), str(tmp_path / "model.pt"))
    os.remove(path)
    model2 = bm.GPTLadder(ModelArgs(**kw)).to(torch.bfloat16)
    load_checkpoint(model2, str(tmp_path))
    assert all(torch.equal(a, b) for a, b in zip(model.parameters(), model2.parameters()))
    bad = dict(hf)
    del bad["model.layers.3.mlp.up_proj.weight"]
    with pytest.raises(KeyError):
        load_checkpoint(model, bad)
    with pytest.raises(KeyError):
        load_checkpoint(model, dict(convert_hf_state_dict(hf, SHAPE["n_head"], SHAPE["n_kv"]), extra=torch.zeros(1)))
    # the parallel family's fused block takes the same checkpoints
    par = bm.GPTParallel(ModelArgs(**dict(kw, ladder_layers=None))).to(torch.bfloat16)
    load_checkpoint(par, hf)
    w = par.layers[0].attention.wqkv1.weight
    assert torch.equal(w[: want["layers.0.attention.wqkv.weight"].shape[0]], want["layers.0.attention.wqkv.weight"].to(torch.bfloat16))
    assert torch.equal(par.layers[0].attention.w2.weight, want["layers.0.feed_forward.w2.weight"].to(torch.bfloat16))


@pytest.mark.gpu
@pytest.mark.parametrize("tp,rank,ladder_layers", [(1, 0, [2, 3]), (2, 1, [2, 3]), (2, 0, None), (1, 0, [1])])
def test_hip_model_serves_a_loaded_hf_checkpoint(tmp_path, tp, rank, ladder_layers):
    """A synthetic HF Llama-Ladder checkpoint (head_dim 64) on disk -> load_checkpoint -> prefill + decode on the HIP
    kernels, against the oracle on the same rank's parameters; un-sharded, also against the HF-form restatement."""
    import benchmark as bm
    from gpt_fast.checkpoint import load_checkpoint
    from gpt_fast.config import ModelArgs
    from safetensors.torch import save_file

    shape = dict(n_layer=4, n_head=4, n_kv=2, dim=256, ffn=512, vocab=320)
    hf = random_hf_state_dict(**shape, seed=11, dtype=torch.bfloat16)
    path = str(tmp_path / "model.safetensors")
    save_file(hf, path)
    kw = dict(block_size=64, vocab_size=320, n_layer=4, n_head=4, n_local_heads=2, dim=256, intermediate_size=512,
              rope_base=10000, tp_world_size=tp, tp_rank=rank, shard_vocab=tp > 1, ladder_layers=ladder_layers)
    with torch.device("meta"):
        model = bm.GPTLadder(ModelArgs(**kw))
    model = model.to(dtype=torch.bfloat16).to_empty(device="cuda").eval()
    load_checkpoint(model, path)
    cfg = model.config
    ocfg = O.OracleConfig(block_size=64, vocab_size=320, n_layer=4, n_head=4, n_local_heads=2, dim=256, intermediate_size=512,
                          rope_base=10000, tp_world_size=tp, vocab_shard=cfg.output_rows if tp > 1 else None,
                          ladder_layers=cfg.ladder_layers)
    P = dict(model.state_dict())
    B, T, new = 2, 21, 6
    g = torch.Generator(device="cuda").manual_seed(2)
    prompt = torch.randint(0, 320, (T,), device="cuda", generator=g)
    with torch.no_grad():
        model.setup_caches(B, T + new)
        ref_tok, ref_logits = O.generate(ocfg, P, prompt, new, B, "ladder")
        rows = prompt.view(1, -1).repeat(B, 1)
        logits = model(rows, torch.arange(T, device="cuda"))
        full_prefill = logits.clone()
        pos = torch.tensor([T], dtype=torch.int32, device="cuda")
        for i in range(new):
            want = ref_logits[i].float()
            assert ((logits[:, -1].float() - want).abs().max() / want.abs().max()).item() <= 2e-2, i
            if i + 1 < new:
                logits = model(ref_tok[:, i:i + 1].contiguous(), pos)
                pos += 1
        model.check_device_errors()
    assert (model._fused_step(B) is not None) == (cfg.ladder_layers is None)
    if tp == 1:
        hf32 = {k: v.float() for k, v in hf.items()}
        want = hf_ladder_forward(hf32, rows.cpu(), 4, 4, 2, 10000.0, 1e-5, ladder_layers)
        got = full_prefill.float().cpu()
        assert ((got - want).abs().max() / want.abs().max()).item() <= 3e-2
