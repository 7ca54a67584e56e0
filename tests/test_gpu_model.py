"""End-to-end parity on a real MI355X: the gpt_fast models on the HIP kernels against the oracle
(oracle/ladder_oracle.py run in eager PyTorch on the same device) on IDENTICAL weights -- the
product model's own parameters are handed to the oracle as its parameter dict -- and identical
token inputs.

What is asserted, per decode step and for prefill:
  * logits: max |hip - oracle| / max |oracle| <= 2e-2 (the stated tolerance), measured when both
    sides are fed the same tokens (teacher forcing on the oracle's stream), so an early flipped
    token cannot hide or fake later agreement;
  * tokens: the HIP argmax equals the oracle's, except at steps where the oracle's own top
    candidates are within 2 bf16 ulp of each other: with N(0, 0.02) weights and gains the logits
    are tiny and near-tied, and bf16 rounding of differently-ordered fp32 sums legitimately picks
    either.  There the HIP token must be one of those tied candidates.  Free-running generations
    must be identical up to the first such near-tie;
  * the captured hipGraph step replays bit-identically to eager launches."""
import gc
import os

import pytest
import torch

from oracle import ladder_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _release_device_memory():
    """Every test builds its own model (up to 101 GB): hand the memory back before the next one."""
    yield
    gc.collect()
    torch.cuda.empty_cache()

DEV = "cuda"
BF = torch.bfloat16
REL_TOL = 2e-2


_PROGRESS_LOG = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out", "test_progress.log")


def progress(msg):
    """Long tests say where they are, and leave their statistics, in a file (pytest's capture holds
    stdout and stderr back until a test has finished)."""
    print(msg)
    try:
        os.makedirs(os.path.dirname(_PROGRESS_LOG), exist_ok=True)
        with open(_PROGRESS_LOG, "a") as f:
            f.write(msg + "\n")
    except OSError:
        pass


def build(family, seed=0, **cfg_kw):
    import benchmark as bm
    from gpt_fast.config import ModelArgs

    cls = {"ladder": bm.GPTLadder, "dense": bm.GPTDense, "desync": bm.GPTDesync, "parallel": bm.GPTParallel}[family]
    with torch.device("meta"):
        model = cls(ModelArgs(**cfg_kw))
    model = model.to(dtype=BF).to_empty(device=DEV)
    with torch.no_grad():
        bm.init_weights(model, seed)
    return model.eval()


def oracle_cfg(c) -> O.OracleConfig:
    return O.OracleConfig(block_size=c.block_size, vocab_size=c.vocab_size, n_layer=c.n_layer, n_head=c.n_head,
                          dim=c.dim, intermediate_size=c.intermediate_size, n_local_heads=c.n_local_heads,
                          rope_base=c.rope_base, norm_eps=c.norm_eps, rope_scaling=c.rope_scaling,
                          reduce_pattern=c.reduce_pattern, force_disable_last_all_reduce=c.force_disable_last_all_reduce,
                          ladder_layers=c.ladder_layers,
                          tp_world_size=c.tp_world_size, vocab_shard=c.output_rows if c.shard_vocab else None)


def rel_err(got, want):
    return ((got.float() - want.float()).abs().max() / want.float().abs().max()).item()


def near_tie_ok(ref_logits, tok, ulps=2):
    """ref_logits [B, V]; tok [B]: is the oracle's logit at `tok` within `ulps` bf16 steps of its maximum?"""
    top = ref_logits.float().max(-1).values
    at = ref_logits.float().gather(-1, tok.long().view(-1, 1)).squeeze(-1)
    ulp = torch.maximum(top.abs(), torch.tensor(1e-30, device=top.device)).log2().floor().exp2() * 2.0 ** -7
    return (top - at) <= ulps * ulp


@torch.no_grad()
def run_parity(model, family, B, T, new, seed=1, check_graph=True, fused=None):
    """Prefill + (new - 1) decode steps, HIP vs oracle.  Returns a dict of statistics.
    fused: True / False selects the persistent one-kernel decode step or the per-op kernels for the
    ladder family at batch <= 2 (None: the model's default)."""
    import benchmark as bm

    if fused is not None:
        model.use_fused_step = fused
    cfg = model.config
    ocfg = oracle_cfg(cfg)
    P = dict(model.state_dict())          # the very same device tensors
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    prompt = torch.randint(0, cfg.vocab_size, (T,), device=DEV, generator=g)
    model.setup_caches(B, T + new)

    big = cfg.n_layer * cfg.dim >= 80 * 4096
    if big:
        progress(f"{family} B={B} T={T} new={new}: oracle generation")
    ref_tok, ref_logits = O.generate(ocfg, P, prompt, new, B, family)            # free-running oracle
    if big:
        progress("teacher-forced HIP run")
    # --- teacher-forced HIP run on the oracle's token stream
    rows = prompt.view(1, -1).repeat(B, 1)
    logits = model(rows, torch.arange(T, device=DEV))
    assert logits.shape == (B, T, cfg.output_rows)
    errs = [rel_err(logits[:, -1], ref_logits[0])]
    hip_tok = [model.greedy_next(logits).clone()]
    pos = torch.tensor([T], dtype=torch.int32, device=DEV)
    for i in range(new - 1):
        logits = model(ref_tok[:, i:i + 1].contiguous(), pos)
        errs.append(rel_err(logits[:, -1], ref_logits[i + 1]))
        hip_tok.append(model.greedy_next(logits).clone())
        pos += 1
    hip_tok = torch.cat(hip_tok, dim=1)
    exact = hip_tok == ref_tok
    tied = torch.stack([near_tie_ok(ref_logits[i], hip_tok[:, i]) for i in range(new)], dim=1)
    stats = dict(max_rel_err=max(errs), exact_frac=exact.float().mean().item(), all_exact_or_tied=bool((exact | tied).all()))

    # --- free-running HIP generation through the benchmark loop (eager), vs the oracle's stream
    if big:
        progress("free-running HIP generation")
    empty = torch.empty(B, T + new, dtype=torch.int64, device=DEV)
    y, _, _ = bm.generate(model, prompt, new, B, empty, greedy=True)
    free = y[:, T:].to(torch.int32)
    same = (free == ref_tok).all(0)
    first_div = int((~same).nonzero()[0]) if not same.all() else new
    stats["first_divergence"] = first_div
    if first_div < new:   # the step where they part must be a near-tie for the oracle
        stats["divergence_is_near_tie"] = bool(near_tie_ok(ref_logits[first_div], free[:, first_div]).all())
    else:
        stats["divergence_is_near_tie"] = True

    # --- hipGraph replay == eager, bit for bit, on several replays
    if check_graph:
        if big:
            progress("hipGraph replay")
        dg = bm.get_cuda_graphs_for_decode(model, prompt, B, new, y[:, T:T + 1].to(torch.int32), greedy=True)
        # re-prefill: the warm-up steps inside graph construction wrote cache slots at position T
        model(rows, torch.arange(T, device=DEV))
        dg.reset(y[:, T:T + 1].to(torch.int32))
        for _ in range(new - 1):
            dg.replay()
        torch.cuda.synchronize()
        stats["graph_equals_eager"] = bool(torch.equal(dg.history[:, : new - 1], free[:, 1:]))
    fs = getattr(model, "_fused", {}).get(B) if getattr(model, "use_fused_step", False) else None
    stats["fused_step_used"] = fs is not None
    if fs is not None:
        assert not fs.failed(), "a device-wide barrier of the fused decode step timed out"
    return stats


def check(stats, min_exact=0.7):
    assert stats["max_rel_err"] <= REL_TOL, stats
    assert stats["all_exact_or_tied"], stats
    assert stats["exact_frac"] >= min_exact, stats
    assert stats["divergence_is_near_tie"], stats
    assert stats.get("graph_equals_eager", True), stats


TINY = dict(block_size=64, vocab_size=512, n_layer=3, n_head=4, n_local_heads=2, dim=256, intermediate_size=512,
            rope_base=10000)


@pytest.mark.parametrize("B", [1, 2])
@pytest.mark.parametrize("fused", [True, False])
def test_tiny_ladder_fused_and_per_op_decode(B, fused):
    stats = run_parity(build("ladder", **TINY), "ladder", B=B, T=20, new=12, fused=fused)
    print(B, fused, stats)
    check(stats)
    assert stats["fused_step_used"] == fused


@pytest.mark.parametrize("B", [1, 3, 6])
@pytest.mark.parametrize("mode", ["plain", "two_streams"])
def test_tiny_ladder_per_op_decode_modes(B, mode):
    """The per-op decode path of the ladder model: one stream (the default), or the attention and the MLP chain
    of a block on two streams."""
    model = build("ladder", **dict(TINY, dim=512, n_head=8, n_local_heads=2, intermediate_size=640))
    model.overlap_modules = mode == "two_streams"
    stats = run_parity(model, "ladder", B=B, T=20, new=12, fused=False)
    print(B, mode, stats)
    check(stats)


def test_tiny_ladder_mlp_chain_as_a_parallel_graph_branch():
    """Above 16 sequences the MLP chain can run beside the attention chain as a second branch of the captured graph
    (the default from 33 sequences on): same tokens and logits as the oracle, replays equal to eager."""
    model = build("ladder", **dict(TINY, dim=512, n_head=8, n_local_heads=2, intermediate_size=640))
    model.two_chains_from = 17
    stats = run_parity(model, "ladder", B=20, T=20, new=12, fused=False)
    print(stats)
    check(stats)


def test_tiny_ladder_fused_head_dim_128_many_kv_heads():
    kw = dict(TINY, block_size=128, n_head=8, n_local_heads=2, dim=1024, intermediate_size=768, n_layer=2,
              vocab_size=1000)
    stats = run_parity(build("ladder", **kw), "ladder", B=2, T=70, new=10, fused=True)
    print(stats)
    check(stats)
    assert stats["fused_step_used"]


@pytest.mark.parametrize("B", [1, 2])
def test_fused_step_several_attention_workgroups_ragged_merge_shares(B):
    # a cache of 360 slots gives three attention workgroups; 8 heads x 64 / 2 = 256 (B = 1) or 512 output pairs
    # are merged in shares of 86, 86, 84 (171, 171, 170) by the attention workgroups; the key range splits unevenly
    kw = dict(TINY, block_size=360, n_head=8, n_local_heads=2, dim=512, intermediate_size=640, n_layer=3)
    stats = run_parity(build("ladder", **kw), "ladder", B=B, T=330, new=10, fused=True)
    print(B, stats)
    check(stats)
    assert stats["fused_step_used"]


@torch.no_grad()
def test_fused_step_exchange_tags_wrap_around():
    # every exchanged word carries a 16-bit tag of the slot that wrote it; a 3-layer step uses 5 tags, so 65535 tags
    # are used up after 13107 launches.  The step is deterministic: the same token at the same position must give
    # the same logits, bit for bit, before the wrap, across it and after it, and no wait may time out.
    model = build("ladder", **TINY)
    model.use_fused_step = True
    T = 20
    model.setup_caches(1, T + 4)
    g = torch.Generator(device=DEV)
    g.manual_seed(3)
    prompt = torch.randint(0, TINY["vocab_size"], (1, T), device=DEV, generator=g)
    model(prompt, torch.arange(T, device=DEV))
    tok = torch.tensor([[7]], dtype=torch.int32, device=DEV)
    pos = torch.tensor([T], dtype=torch.int32, device=DEV)
    first = model(tok, pos).clone()
    fs = model._fused[1]
    for i in range(13400):
        out = model(tok, pos)
        if i in (13000, 13100, 13110, 13399):
            assert torch.equal(out, first), i
    torch.cuda.synchronize()
    assert not fs.failed()


@pytest.mark.parametrize("family", ["ladder", "dense", "desync", "parallel"])
@pytest.mark.parametrize("B", [1, 3])
def test_tiny_all_families(family, B):
    kw = dict(TINY)
    if family == "desync":
        kw.update(reduce_pattern=[{"attention": True, "mlp": False}, {"attention": False, "mlp": True},
                                  {"attention": False, "mlp": False}], tp_world_size=2)
    stats = run_parity(build(family, **kw), family, B=B, T=20, new=12)
    print(family, B, stats)
    check(stats)


@pytest.mark.parametrize("family", ["ladder", "parallel"])
def test_tiny_rank_shard_with_vocab_shard(family):
    kw = dict(TINY, n_head=8, n_local_heads=4, dim=512, intermediate_size=1024, tp_world_size=4, shard_vocab=True)
    model = build(family, **kw)
    assert model.output.weight.shape == (128, 512) and model.layers[0].attention.wo.weight.shape == (512, 128)
    stats = run_parity(model, family, B=2, T=33, new=8)
    print(family, stats)
    check(stats)


def test_semi_compiled_nonzero_rank_drops_the_residual():
    """gpt_dense_TP.py:256-257: on ranks other than 0 the residual is not added."""
    kw = dict(TINY, n_layer=2, tp_world_size=2, tp_rank=1, semi_compiled_model=True)
    model = build("dense", **kw)
    model.setup_caches(1, 16)
    P = dict(model.state_dict())
    ocfg = oracle_cfg(model.config)
    idx = torch.tensor([[5, 7, 300, 2]], device=DEV)
    pos = torch.arange(4, device=DEV)
    got = model(idx, pos)
    caches = O.setup_caches(ocfg, 1, 16, BF, DEV)
    x = torch.nn.functional.embedding(idx, P["tok_embeddings.weight"])
    for i in range(2):
        x = O.attention(ocfg, P, i, O.rms_norm(x, P[f"layers.{i}.attention_norm.weight"], 1e-5), caches,
                        caches.freqs_cis[pos], caches.causal_mask[pos], pos)
        x = O.feed_forward(ocfg, P, i, O.rms_norm(x, P[f"layers.{i}.ffn_norm.weight"], 1e-5))
    want = torch.nn.functional.linear(O.rms_norm(x, P["norm.weight"], 1e-5), P["output.weight"])
    assert rel_err(got, want) <= REL_TOL


def test_block_level_api_matches_oracle_block():
    """LadderTransformerBlock.forward with the reference's signature (gpt_ladder_TP.py:312-358)."""
    model = build("ladder", **TINY)
    model.setup_caches(2, 16)
    cfg, ocfg = model.config, oracle_cfg(model.config)
    P = dict(model.state_dict())
    g = torch.Generator(device=DEV)
    g.manual_seed(5)
    mk = lambda: (torch.randn(2, 6, cfg.dim, device=DEV, generator=g) * 0.1).to(BF)
    pa, pm, r = mk(), mk(), mk()
    pos = torch.arange(6, device=DEV)
    fc, mask = model.freqs_cis[pos], model.causal_mask[None, None, pos]
    a, m, r2, ha, hm = model.layers[1](pa, pm, r, None, None, pos, fc, mask)
    caches = O.setup_caches(ocfg, 2, 16, BF, DEV)
    a_ref, m_ref, r_ref = O.ladder_block(ocfg, P, 1, pa, pm, r, caches, caches.freqs_cis[pos], caches.causal_mask[pos], pos)
    assert ha is None and hm is None
    assert torch.equal(r2, r_ref)
    assert rel_err(a, a_ref) <= REL_TOL and rel_err(m, m_ref) <= REL_TOL
    assert torch.equal(model.layers[1].attention.kv_cache.k_cache[:, :, :6], caches.k[1][:, :, :6])


def test_prefill_last_logits_only_equals_full():
    model = build("ladder", **TINY)
    model.setup_caches(2, 24)
    idx = torch.randint(0, 512, (2, 17), device=DEV)
    pos = torch.arange(17, device=DEV)
    full = model(idx, pos)[:, -1].clone()
    model.last_logits_only = True
    last = model(idx, pos)
    assert last.shape == (2, 1, 512)
    # the two runs push different row counts through the lm_head (34 rows: matrix-core GEMM, 2 rows:
    # GEMV), i.e. different fp32 summation orders: equal up to one bf16 rounding step in a few places
    got, want = last[:, 0].float(), full.float()
    ulp = want.abs().clamp_min(1e-30).log2().floor().exp2() * 2.0 ** -7
    assert bool(((got - want).abs() <= ulp).all()) and (got == want).float().mean().item() >= 0.9


# ---------------------------------------------------------------------------------------------------
# every instance of the one-kernel step, its limits and its failure word
# ---------------------------------------------------------------------------------------------------

STEP_INSTANCES = [(1, 128, 8), (2, 128, 8), (1, 128, 4), (2, 128, 4), (1, 64, 4), (2, 64, 4), (1, 128, 16), (1, 64, 2),
                  (2, 64, 2), (1, 128, 2), (1, 128, 1), (1, 64, 1), (1, 64, 8)]


@pytest.mark.parametrize("B,hd,G", STEP_INSTANCES)
@pytest.mark.parametrize("fp8", [False, True])
def test_fused_step_every_instance(B, hd, G, fp8):
    """One parity run per (batch, head_dim, q heads per kv head) the step kernel is built for: multi-head
    attention (G = 1, where the shared-memory carve-up has an odd number of per-head scalars), grouped
    queries up to 16 per kv head, both head sizes; on bf16 weights and on weight-only e4m3 projections
    (lr_ladder_decode_step_fp8, against the oracle on the same quantised weights and scales)."""
    from gpt_fast.quantize import quantize_model_fp8

    hkv = 1 if G == 16 else 2
    kw = dict(TINY, block_size=128, n_head=hkv * G, n_local_heads=hkv, dim=hkv * G * hd, intermediate_size=512,
              n_layer=2)
    model = build("ladder", **kw)
    if fp8:
        quantize_model_fp8(model)
    stats = run_parity(model, "ladder", B=B, T=40, new=6, fused=True)
    print(B, hd, G, fp8, stats)
    check(stats)
    assert stats["fused_step_used"]


def test_fused_step_is_refused_unless_every_workgroup_can_be_resident():
    """The step launches one workgroup per compute unit and they wait for each other: the library reports how many
    workgroups of the instance the device can hold for a descriptor (occupancy x compute units), refuses the
    launch below one per compute unit, and reports 0 for shapes the step does not serve."""
    import ctypes

    from gpt_fast import _hip

    cus = torch.cuda.get_device_properties(0).multi_processor_count
    lib = _hip.load()
    big = build("ladder", **dict(TINY, block_size=2200, n_head=8, n_local_heads=1, dim=1024, intermediate_size=3584,
                                 n_layer=1))     # the rank shard's head layout: the 70B instance, LDS sized by ffn
    big.setup_caches(1, 2112)
    fs = _hip.FusedLadderStep(big, 1)
    assert fs.supported and fs.resident >= cus
    assert lib.lr_ladder_step_resident_workgroups(ctypes.byref(fs.desc), 1) == fs.resident      # remembered per device
    assert lib.lr_ladder_step_resident_workgroups(ctypes.byref(fs.desc), 3) == 0                 # no instance for batch 3
    # fewer q/k/v rows than compute units: some workgroup would own no row of the projection that orders the
    # exchange arrays -- left to the per-op kernels
    thin = build("ladder", **dict(TINY, n_head=1, n_local_heads=1, dim=64, intermediate_size=512, n_layer=1))
    thin.setup_caches(1, 64)
    assert (1 + 2) * 64 < cus
    assert not _hip.FusedLadderStep(thin, 1).supported


def test_fused_step_head_dim_64_longest_key_range_per_workgroup():
    """head_dim 64 with a cache of 8160 slots: 16 attention workgroups of 510 keys each, the most a
    workgroup's score tiles cover (2 x 8 waves x 32 keys = 512).  Beyond that the step must refuse."""
    from gpt_fast import _hip

    kw = dict(TINY, block_size=9216, n_head=4, n_local_heads=2, dim=256, intermediate_size=512, n_layer=2)
    model = build("ladder", **kw)
    stats = run_parity(model, "ladder", B=1, T=8150, new=6, fused=True, check_graph=False)
    print(stats)
    check(stats)
    assert stats["fused_step_used"]
    model.max_seq_length = -1
    model.setup_caches(1, 8200)      # 8200 / 16 = 513 keys per workgroup: not covered
    assert not _hip.FusedLadderStep(model, 1).supported


@torch.no_grad()
@pytest.mark.parametrize("fused", [True, False])
def test_position_out_of_range_is_reported_not_clamped(fused):
    """A decode step at a position beyond the cache writes nothing and leaves an error word behind
    (the reference raises an index error at utils.py:55); both decode paths behave the same."""
    from gpt_fast import _hip

    model = build("ladder", **TINY)
    model.use_fused_step = fused
    T = 20
    model.setup_caches(1, T + 4)     # cache of 24 slots
    prompt = torch.randint(0, TINY["vocab_size"], (1, T), device=DEV)
    model(prompt, torch.arange(T, device=DEV))
    tok = torch.tensor([[7]], dtype=torch.int32, device=DEV)
    good = model(tok, torch.tensor([T], dtype=torch.int32, device=DEV)).clone()
    model.check_device_errors()
    caches = [b.attention.kv_cache.k_cache.clone() for b in model.layers]
    model(tok, torch.tensor([24], dtype=torch.int32, device=DEV))
    with pytest.raises(_hip.LadderHipError):
        model.check_device_errors()
    assert all(torch.equal(c, b.attention.kv_cache.k_cache) for c, b in zip(caches, model.layers))
    if fused:
        fs = model._fused_step(1)
        assert fs.fail_code() == _hip.DEV_POS_RANGE
        # out of service until it is initialised again
        model(tok, torch.tensor([T], dtype=torch.int32, device=DEV))
        assert fs.fail_code() == _hip.DEV_POS_RANGE
        fs.reset()
    again = model(tok, torch.tensor([T], dtype=torch.int32, device=DEV))
    model.check_device_errors()
    assert torch.equal(again, good)


def test_setup_caches_refuses_more_positions_than_the_rope_table_has():
    model = build("ladder", **TINY)        # block_size 64
    with pytest.raises(ValueError):
        model.setup_caches(1, 65)
    model.setup_caches(1, 64)


# ---------------------------------------------------------------------------------------------------
# the benchmark harness: graphs for prefill and decode, the command-line entry, sampling
# ---------------------------------------------------------------------------------------------------

@torch.no_grad()
@pytest.mark.parametrize("B", [1, 3])
def test_generate_using_cuda_graphs_equals_eager_generate(B):
    """benchmark.py:167-225, 253-305: prefill graph + decode graph replay produce the tokens of the eager loop."""
    import benchmark as bm

    model = build("ladder", **TINY)
    T, new = 20, 12
    model.setup_caches(B, T + new)
    g = torch.Generator(device=DEV)
    g.manual_seed(4)
    prompt = torch.randint(0, TINY["vocab_size"], (T,), device=DEV, generator=g)
    empty = torch.empty(B, T + new, dtype=torch.int64, device=DEV)
    want, _, _ = bm.generate(model, prompt, new, B, empty, greedy=True)
    want = want.clone()

    pg, static_x, static_pos, static_next = bm.get_cuda_graphs_for_prefill(model, prompt, B, greedy=True)
    first = torch.zeros(B, 1, dtype=torch.int32, device=DEV)
    dg = bm.get_cuda_graphs_for_decode(model, prompt, B, new, first, greedy=True)
    for _ in range(2):   # a graph is replayed many times in the benchmark: the second generation must equal the first
        out = torch.empty(B, T + new, dtype=torch.int64, device=DEV)
        got, dec_s, pre_s = bm.generate_using_cuda_graphs(pg, static_x, static_pos, static_next, dg, prompt, B, out, new)
        assert torch.equal(got, want)
        assert dec_s > 0 and pre_s > 0
    model.check_device_errors()


def test_benchmark_main_prints_the_reference_metric_lines(tmp_path, capsys, monkeypatch):
    """benchmark.py:381-488: the command-line entry on a small registered shape, with --json."""
    import json

    import benchmark as bm
    from gpt_fast.config import REGISTRIES
    from gpt_fast.utils import _get_model_size

    monkeypatch.setitem(REGISTRIES["ladder"], "tiny-test", dict(TINY))
    out = tmp_path / "r.json"
    res = bm.main("gpt_ladder:tiny-test", prompt_length=16, num_samples=2, max_new_tokens=8, batch_size=2, top_k=5,
                  temperature=0.8, compile=False, device="cuda", use_cuda_graphs=True, greedy=True, seed=0,
                  json_path=out, warmup=1)
    text = capsys.readouterr().out
    for line in ("Using device=cuda", "Time to load model", "Compilation time", "Time for inference 2",
                 "Tokens per second per user", "Total tokens per second", "Decode latency", "Prefill latency",
                 "Bandwidth achieved", "FLOPS achieved", "Batch Size: 2", "Prompt Length: 16", "Generated tokens: 8",
                 "Average decode latency", "Average prefill latency", "Average tokens/sec/user", "Average tokens/sec:",
                 "Memory used"):
        assert line in text, line
    saved = json.loads(out.read_text())
    assert saved["batch_size"] == 2 and len(saved["tokens"]) == 8 and saved["ms_per_token"] > 0
    assert saved["tokens"] == res["tokens"]
    # the eager (no graph) path of main and the sampling path with the reference's default flags
    res2 = bm.main("gpt_ladder:tiny-test", prompt_length=16, num_samples=1, max_new_tokens=8, batch_size=2, top_k=5,
                   temperature=0.8, compile=False, device="cuda", use_cuda_graphs=False, greedy=True, seed=0, warmup=0)
    assert res2["tokens"] == res["tokens"]
    res3 = bm.main("gpt_ladder:tiny-test", prompt_length=16, num_samples=1, max_new_tokens=8, batch_size=2, top_k=5,
                   temperature=0.8, compile=True, device="cuda", greedy=False, seed=0, warmup=0)
    assert len(res3["tokens"]) == 8 and all(0 <= t < TINY["vocab_size"] for t in res3["tokens"])
    # _get_model_size (utils.py:400-409) leaves the embedding table out
    model = build("ladder", **TINY)
    size, params = _get_model_size(model)
    want = sum(p.numel() for n, p in model.named_parameters() if not n.startswith("tok_embeddings"))
    assert params == want and size == 2 * want


@torch.no_grad()
def test_sample_goes_through_the_device_sampler_and_matches_the_oracle():
    """benchmark.py:58-77 via sample() -> model.sample_next -> lr_sample_topk, with the same Exp(1) draws."""
    import benchmark as bm

    model = build("ladder", **TINY)
    model.setup_caches(3, 32)
    idx = torch.randint(0, TINY["vocab_size"], (3, 9), device=DEV)
    logits = model(idx, torch.arange(9, device=DEV))
    torch.manual_seed(11)
    noise = torch.empty(3, TINY["vocab_size"], dtype=BF, device=DEV).exponential_(1)
    torch.manual_seed(11)
    tok, probs = bm.sample(logits, temperature=0.7, top_k=7, model=model)
    want_tok, want_probs = O.sample_topk(logits[:, -1], noise, 0.7, 7)
    assert tok.dtype == torch.int32 and tok.shape == (3, 1) and torch.equal(tok, want_tok)
    assert int((probs > 0).sum(-1).max()) <= 7 + 2 and rel_err(probs, want_probs) <= 2.0 ** -7
    # greedy flag: the device argmax
    tok_g, none = bm.sample(logits, greedy=True, model=model)
    assert none is None and torch.equal(tok_g, torch.argmax(logits[:, -1], -1, keepdim=True).to(torch.int32))


# ---------------------------------------------------------------------------------------------------
# weight-only fp8 decode
# ---------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("family", ["ladder", "dense", "parallel"])
def test_tiny_models_with_fp8_weights(family):
    from gpt_fast.quantize import quantize_model_fp8

    model = quantize_model_fp8(build(family, **dict(TINY, dim=256, intermediate_size=512)))
    assert model.output.weight.dtype == torch.float8_e4m3fn and "layers.0.attention.wo.scales" in model.state_dict()
    stats = run_parity(model, family, B=2, T=20, new=10)
    print(family, stats)
    check(stats)
    assert stats["fused_step_used"] == (family == "ladder")


@pytest.mark.parametrize("B", [1, 2])
@torch.no_grad()
def test_tiny_ladder_fp8_one_kernel_step_against_the_per_op_kernels(B):
    """lr_ladder_decode_step_fp8 and the per-op fp8 kernels on the same quantised model and the same tokens: logits
    within the tolerance of two summation orders, the same KV cache rows; a model whose lm_head stays bf16 is not
    taken by the one-kernel step; packing the scales behind the weights leaves the values as they were."""
    from gpt_fast.quantize import quantize_model_fp8

    model = quantize_model_fp8(build("ladder", **TINY))
    w_before = model.layers[1].feed_forward.w1.weight.clone()
    s_before = model.layers[1].feed_forward.w1.scales.clone()
    model.setup_caches(B, 32)
    g = torch.Generator(device=DEV)
    g.manual_seed(5)
    toks = torch.randint(0, 512, (B, 12), device=DEV, generator=g)

    def steps(fused):
        model.use_fused_step = fused
        out = [model(toks[:, :6], torch.arange(6, device=DEV)).clone()]
        for t in range(6, 12):
            out.append(model(toks[:, t:t + 1], torch.tensor([t], device=DEV)).clone())
        model.check_device_errors()
        kv = model.layers[-1].attention.kv_cache
        return out, kv.k_cache[:B, :, :12].clone(), kv.v_cache[:B, :, :12].clone()

    per_op, kp, vp = steps(False)
    one, ko, vo = steps(True)
    assert model._fused[B] is not None and model._fused[B].fp8
    for a, b in zip(per_op, one):
        assert rel_err(b, a) <= REL_TOL
    assert rel_err(ko, kp) <= REL_TOL and rel_err(vo, vp) <= REL_TOL
    w1 = model.layers[1].feed_forward.w1
    assert torch.equal(w1.weight.view(torch.uint8), w_before.view(torch.uint8)) and torch.equal(w1.scales, s_before)
    assert w1.scales.data_ptr() == w1.weight.data_ptr() + w1.weight.numel()

    mixed = quantize_model_fp8(build("ladder", **TINY), include_output=False)
    mixed.setup_caches(B, 32)
    mixed(toks[:, :6], torch.arange(6, device=DEV))
    mixed(toks[:, 6:7], torch.tensor([6], device=DEV))
    assert mixed._fused[B] is None


@pytest.mark.parametrize("B", [1, 2, 8])
def test_ladder_70b_tp8_shard_shape_with_fp8_weights(B):
    """The 70B rank shard's matrices (12 layers) in the weight-only fp8 form: prefill (expanded weights, matrix-core
    GEMM) and decode (batch 1 and 2: the one-kernel fp8 step; batch 8: the fp8 bands) against the oracle on the same
    fp8 weights and scales."""
    from gpt_fast.quantize import quantize_model_fp8

    model = quantize_model_fp8(build("ladder", **shape_kw("ladder-70b-tp8", 12)))
    stats = run_parity(model, "ladder", B=B, T=512, new=24)
    report(f"fp8 weights, cfg3 shape, 12 layers, B={B}", stats)
    check(stats)


@pytest.mark.parametrize("B", [1, 8])
def test_ladder_70b_tp8_shard_config3_full_with_fp8_weights(B):
    """Config 3 at its full size (80 layers, prompt 2048) in the weight-only fp8 form: batch 1 through the
    one-kernel step on e4m3 weights, batch 8 through the fp8 bands."""
    from gpt_fast.quantize import quantize_model_fp8

    progress(f"cfg3 fp8 B={B}: building")
    model = quantize_model_fp8(build("ladder", **shape_kw("ladder-70b-tp8")))
    stats = run_parity(model, "ladder", B=B, T=2048, new=32)
    report(f"fp8 weights, cfg3 ladder-70b-tp8, 80 layers, B={B}", stats)
    check(stats)
    assert stats["fused_step_used"] == (B == 1)


# ---------------------------------------------------------------------------------------------------
# token identity with teeth: weights under which the greedy token changes from step to step
# ---------------------------------------------------------------------------------------------------

@torch.no_grad()
def init_conditioned(model, seed, head_tail=2.5, branch_gain=0.25):
    """Unit norm gains, N(0, 1 / fan_in) projections, N(0, 1) embeddings: activations of order one in
    every layer, so every layer's arithmetic shows in the logits.  The output projections of the two
    branches (wo, w2) are scaled by `branch_gain`, as in a trained network where a block adds a
    small correction to the residual stream: 160 such corrections still outweigh the embedding in
    the final hidden state, but a one-step rounding difference in one of them is not amplified by
    the 79 layers behind it.  The rows of the lm_head get log-normal lengths: the winning logit
    then usually stands clear of the runner-up by many bf16 steps, while WHICH row wins still
    depends on the sign and size of its dot product with the final hidden state -- the greedy token
    moves from step to step (with N(0, 0.02) weights and gains the benchmark model emits one
    constant token, and "tokens identical" says little)."""
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    for name, p in model.named_parameters():
        if name.endswith("norm.weight"):
            p.fill_(1.0)
        elif name == "tok_embeddings.weight":
            p.normal_(0.0, 1.0, generator=g)
        else:
            gain = branch_gain if name.endswith(("wo.weight", "w2.weight")) else 1.0
            p.normal_(0.0, gain * p.shape[1] ** -0.5, generator=g)
            if name == "output.weight":
                length = torch.exp(head_tail * torch.randn(p.shape[0], 1, device=DEV, generator=g))
                p.mul_(length.to(p.dtype))


def oracle_margins(ref_logits):
    """Per step: (top - runner-up) in bf16 steps of the top logit, minimum over the batch."""
    top2 = ref_logits.float().topk(2, dim=-1).values
    ulp = top2[..., 0].abs().clamp_min(1e-30).log2().floor().exp2() * 2.0 ** -7
    return ((top2[..., 0] - top2[..., 1]) / ulp).min(-1).values


CONDITIONED_PROMPT_SEED = 21   # a prompt for which the oracle's token stream moves (asserted below)


@torch.no_grad()
@pytest.mark.parametrize("name,B,T", [("ladder-70b-tp8", 1, 2048), ("ladder-70b-tp8", 8, 2048), ("ladder-8b", 16, 1024)])
def test_tokens_on_conditioned_weights(name, B, T):
    """The 70B rank shard (batch 1: the one-kernel step; batch 8: the bands with the attention beside up/gate) and the
    8B model (batch 16: eight kv heads per rank, the attention items of all of them beside the up/gate bands) at
    their full size with well-conditioned weights, where the oracle's greedy tokens change from step to step, so
    that "tokens identical" can fail.

    With activations of order one in all 80 layers bf16 arithmetic is itself noisy: the eager bf16
    oracle differs from the SAME oracle run in fp32 by ~1e-1 of the largest logit, and two bf16
    implementations that differ in one rounding decorrelate to that level.  So the yardstick is
    the fp32 run, and what is asserted is
      * the HIP logits are no farther from the fp32 logits than the eager bf16 reference is (x 1.5);
      * at every step where the reference's choice is robust to its own bf16 error -- its margin
        over the runner-up exceeds twice its distance to the fp32 logits -- the HIP token is
        IDENTICAL, with no tie exemption; such steps must be the majority and their tokens must
        vary;
      * free-running generation equals the oracle's up to the first step that is not robust, and
        the hipGraph replay equals the eager generation token for token."""
    import benchmark as bm

    new = 48
    model = build("ladder", **shape_kw(name))
    init_conditioned(model, seed=0)
    cfg, ocfg = model.config, oracle_cfg(model.config)
    P = dict(model.state_dict())
    g = torch.Generator(device=DEV)
    g.manual_seed(CONDITIONED_PROMPT_SEED)
    prompt = torch.randint(0, cfg.vocab_size, (T,), device=DEV, generator=g)
    model.setup_caches(B, T + new)
    progress(f"conditioned weights {name} B={B}: oracle generation (bf16, then fp32 on the same tokens)")
    ref_tok, ref_logits = O.generate(ocfg, P, prompt, new, B, "ladder")
    P32 = {k: v.float() for k, v in P.items()}
    _, exact_logits = O.generate(ocfg, P32, prompt, new, 1, "ladder", forced=ref_tok[:1])
    del P32
    exact_logits = exact_logits.expand(new, B, -1)
    oracle_err = max(rel_err(ref_logits[i], exact_logits[i]) for i in range(new))
    top2 = ref_logits.float().topk(2, dim=-1).values                            # [new, B, 2]
    noise = (ref_logits.float() - exact_logits.float()).abs().amax(-1)          # [new, B]
    robust = ((top2[..., 0] - top2[..., 1]) > 2 * noise).T                      # [B, new]
    distinct = len(set(ref_tok[0][robust[0]].tolist()))
    changes = int((ref_tok[0, 1:] != ref_tok[0, :-1]).sum())
    progress(f"oracle: {int(robust[0].sum())}/{new} robust steps with {distinct} distinct tokens, {changes} token changes, "
             f"min margin {oracle_margins(ref_logits).min().item():.1f} bf16 steps")
    assert robust.float().mean().item() >= 0.5 and distinct >= 3 and changes >= 12, "precondition: pick another prompt seed"

    rows = prompt.view(1, -1).repeat(B, 1)
    logits = model(rows, torch.arange(T, device=DEV))
    errs = [rel_err(logits[:, -1], exact_logits[0])]
    forced = [model.greedy_next(logits).clone()]
    pos = torch.tensor([T], dtype=torch.int32, device=DEV)
    for i in range(new - 1):
        logits = model(ref_tok[:, i:i + 1].contiguous(), pos)
        errs.append(rel_err(logits[:, -1], exact_logits[i + 1]))
        forced.append(model.greedy_next(logits).clone())
        pos += 1
    forced = torch.cat(forced, dim=1)
    same = forced == ref_tok
    line = (f"conditioned weights {name} B={B}: tokens identical at {float(same.float().mean()):.4f} of all steps, at "
            f"{float(same[robust].float().mean()):.4f} of the robust ones; distance to the fp32 logits: HIP {max(errs):.3e}, "
            f"eager bf16 oracle {oracle_err:.3e}")
    progress(line)
    assert max(errs) <= 1.5 * oracle_err
    assert bool(same[robust].all())

    empty = torch.empty(B, T + new, dtype=torch.int64, device=DEV)
    y, _, _ = bm.generate(model, prompt, new, B, empty, greedy=True)
    free = y[:, T:].to(torch.int32).clone()
    horizon = int((~robust.all(0)).nonzero()[0]) if not robust.all() else new    # first step that is not robust
    assert torch.equal(free[:, :horizon], ref_tok[:, :horizon])

    dg = bm.get_cuda_graphs_for_decode(model, prompt, B, new, free[:, :1].contiguous(), greedy=True)
    model(rows, torch.arange(T, device=DEV))
    dg.reset(free[:, :1].contiguous())
    for _ in range(new - 1):
        dg.replay()
    torch.cuda.synchronize()
    model.check_device_errors()
    assert torch.equal(dg.history[:, : new - 1], free[:, 1:])


# ---------------------------------------------------------------------------------------------------
# the benchmark shapes, at their full size
# ---------------------------------------------------------------------------------------------------

def shape_kw(name, n_layer=None):
    from gpt_fast.config import REGISTRIES

    kw = dict(REGISTRIES["ladder"][name])
    if n_layer is not None:
        kw["n_layer"] = n_layer
    return kw


def report(tag, stats):
    line = (f"{tag}: exact_frac {stats['exact_frac']:.4f}  first_divergence {stats['first_divergence']}  "
            f"max_rel_err {stats['max_rel_err']:.3e}  graph_equals_eager {stats.get('graph_equals_eager')}  "
            f"fused {stats['fused_step_used']}")
    progress(line)


def test_ladder_1b_config1_full():
    """Config 1: Ladder-1B, B=1, 128-token prompt, 32 new tokens (head_dim 64, full vocab)."""
    stats = run_parity(build("ladder", **shape_kw("ladder-1b")), "ladder", B=1, T=128, new=32)
    report("cfg1 ladder-1b B=1", stats)
    check(stats)


def test_ladder_70b_tp8_shard_per_op_kernels_b1():
    stats = run_parity(build("ladder", **shape_kw("ladder-70b-tp8", 12)), "ladder", B=1, T=2048, new=24, fused=False)
    report("cfg3 shape, 12 layers, per-op kernels, B=1", stats)
    check(stats)
    assert not stats["fused_step_used"]


@pytest.mark.parametrize("B", [1, 2, 8, 64])
def test_ladder_70b_tp8_shard_config3_full(B):
    """Config 3: one TP=8 rank shard of Ladder-70B (dim 8192, 80 layers, 8 q / 1 kv heads, FFN 3584,
    vocab shard 16032), prompt 2048, 128 new tokens, at every batch size of the benchmark set
    (plus B = 2, the other batch the one-kernel step serves)."""
    progress(f"cfg3 B={B}: building")
    stats = run_parity(build("ladder", **shape_kw("ladder-70b-tp8")), "ladder", B=B, T=2048, new=128)
    report(f"cfg3 ladder-70b-tp8 B={B}", stats)
    check(stats)


@pytest.mark.parametrize("family,B", [("dense", 2), ("desync", 2), ("parallel", 2), ("dense", 8), ("parallel", 1),
                                      ("parallel", 8), ("parallel", 20)])
def test_variants_on_70b_shard_shape(family, B):
    """The other families on the 70B rank shard's matrices (6 layers) against the oracle; decode runs on the bands of
    lr_linear_multi (parallel family: up/gate beside the attention at 1, 2 and 8 sequences, beside q/k/v at 20)."""
    kw = shape_kw("ladder-70b-tp8", 6)
    if family == "desync":
        # one layer of each kind: no reduce, a reduce after attention (residual / tp), after the MLP, after both
        kw.update(reduce_pattern=[{"attention": False, "mlp": False}, {"attention": True, "mlp": False},
                                  {"attention": False, "mlp": True}, {"attention": True, "mlp": True},
                                  {"attention": False, "mlp": False}, {"attention": False, "mlp": False}],
                  force_disable_last_all_reduce=True)
    stats = run_parity(build(family, **kw), family, B=B, T=300, new=10)
    report(f"{family} on the 70B shard shape, B={B}", stats)
    check(stats)


@pytest.mark.parametrize("family,B", [("dense", 1), ("dense", 8), ("parallel", 1), ("parallel", 8)])
def test_variants_on_70b_shard_shape_at_full_depth(family, B):
    """Dense and parallel blocks (gpt_dense_TP.py:274-284, gpt_parallel_TP.py:214-226) on the 70B rank shard's
    matrices at all 80 layers, prompt 2048: what 80 layers of bf16 rounding do to the logits stays within the bar."""
    progress(f"{family} at 80 layers B={B}: building")
    stats = run_parity(build(family, **shape_kw("ladder-70b-tp8")), family, B=B, T=2048, new=24)
    report(f"{family} on the 70B shard shape, 80 layers, B={B}", stats)
    check(stats)


@pytest.mark.parametrize("family", ["dense", "desync", "parallel"])
@pytest.mark.parametrize("B", [3, 20])
@pytest.mark.parametrize("semi", [False, True])
@torch.no_grad()
def test_variant_decode_on_the_bands_equals_the_single_projection_kernels(family, B, semi):
    """Decode steps of the other families through lr_linear_multi (q/k/v with the RoPE + cache epilogue, up/gate with
    the SwiGLU epilogue; parallel family: up/gate beside the attention up to 16 rows, beside q/k/v above, y + x left to
    the next norm) against the same steps through lr_linear and the separate kernels: the same tokens fed, logits
    within the tolerance of two summation orders, KV caches too.  semi: a rank that carries no residual."""
    kw = dict(TINY, tp_world_size=2, tp_rank=1, semi_compiled_model=semi)
    if family == "desync":
        kw.update(reduce_pattern=[{"attention": True, "mlp": False}, {"attention": False, "mlp": True},
                                  {"attention": False, "mlp": False}])
    model = build(family, **kw)
    model.setup_caches(B, 32)
    g = torch.Generator(device=DEV)
    g.manual_seed(3)
    toks = torch.randint(0, 512, (B, 10), device=DEV, generator=g)

    def steps(rows_from):
        model.band_rows_from = rows_from
        out = [model(toks[:, :6], torch.arange(6, device=DEV)).clone()]
        for t in range(6, 10):
            out.append(model(toks[:, t:t + 1], torch.tensor([t], device=DEV)).clone())
        model.check_device_errors()
        kv = model.layers[-1].attention.kv_cache
        return out, kv.k_cache[:B, :, :10].clone(), kv.v_cache[:B, :, :10].clone()

    plain, kp, vp = steps(10 ** 9)
    bands, kb, vb = steps(1)
    assert torch.equal(plain[0], bands[0])   # prefill does not depend on the switch
    for a, b in zip(plain[1:], bands[1:]):
        assert rel_err(b, a) <= REL_TOL
    assert rel_err(kb, kp) <= REL_TOL and rel_err(vb, vp) <= REL_TOL


def test_parallel_semi_compiled_nonzero_rank_drops_the_residual():
    """gpt_parallel_TP.py:197-199: in the semi-compiled model only rank 0 adds the residual."""
    kw = dict(TINY, n_layer=2, tp_world_size=2, tp_rank=1, semi_compiled_model=True)
    model = build("parallel", **kw)
    model.setup_caches(1, 16)
    P = dict(model.state_dict())
    ocfg = oracle_cfg(model.config)
    idx = torch.tensor([[5, 7, 300, 2]], device=DEV)
    pos = torch.arange(4, device=DEV)
    got = model(idx, pos)
    caches = O.setup_caches(ocfg, 1, 16, BF, DEV)
    x = torch.nn.functional.embedding(idx, P["tok_embeddings.weight"])
    for i in range(2):
        x = O.fused_attention_mlp(ocfg, P, i, O.rms_norm(x, P[f"layers.{i}.attention_norm.weight"], 1e-5), caches,
                                  caches.freqs_cis[pos], caches.causal_mask[pos], pos)
    want = torch.nn.functional.linear(O.rms_norm(x, P["norm.weight"], 1e-5), P["output.weight"])
    assert rel_err(got, want) <= REL_TOL


@pytest.mark.parametrize("B", [1, 16])
def test_ladder_8b_config2_full(B):
    """Config 2: Ladder-8B (dim 4096, 32 layers, 32 q / 8 kv heads, FFN 14336, full vocab), prompt 1024,
    256 new tokens, B = 1 and 16."""
    progress(f"cfg2 B={B}: building")
    stats = run_parity(build("ladder", **shape_kw("ladder-8b")), "ladder", B=B, T=1024, new=256)
    report(f"cfg2 ladder-8b B={B}", stats)
    check(stats)


@torch.no_grad()
def test_ladder_8b_config4_prefill_heavy():
    """Config 4: Ladder-8B, batch 32, prompts of 2048 ids: causal prefill (matrix-core GEMM + attention)
    plus one decode step.  Logits of the last prompt position and of the decode step against the
    oracle; the prefill runs with last_logits_only (the benchmark's setting) and, on the first four
    sequences' worth of rows, is also compared position by position."""
    import benchmark as bm

    B, T = 32, 2048
    progress("cfg4: building")
    model = build("ladder", **shape_kw("ladder-8b"))
    cfg, ocfg = model.config, oracle_cfg(model.config)
    P = dict(model.state_dict())
    g = torch.Generator(device=DEV)
    g.manual_seed(1)
    prompt = torch.randint(0, cfg.vocab_size, (T,), device=DEV, generator=g)
    model.setup_caches(B, T + 2)
    progress("cfg4: oracle prefill + 1 step")
    ref_tok, ref_logits = O.generate(ocfg, P, prompt, 2, B, "ladder")
    rows = prompt.view(1, -1).repeat(B, 1)
    model.last_logits_only = True
    progress("cfg4: HIP prefill")
    logits = model(rows, torch.arange(T, device=DEV))
    assert logits.shape == (B, 1, cfg.output_rows)
    e0 = rel_err(logits[:, -1], ref_logits[0])
    t0 = model.greedy_next(logits).clone()
    pos = torch.tensor([T], dtype=torch.int32, device=DEV)
    logits = model(ref_tok[:, :1].contiguous(), pos)
    e1 = rel_err(logits[:, -1], ref_logits[1])
    t1 = model.greedy_next(logits).clone()
    model.check_device_errors()
    progress(f"cfg4: max_rel_err prefill {e0:.3e} decode {e1:.3e}")
    print(f"cfg4 ladder-8b B=32 T=2048: max_rel_err prefill {e0:.3e}, decode step {e1:.3e}")
    assert e0 <= REL_TOL and e1 <= REL_TOL
    for i, t in enumerate((t0, t1)):
        ok = (t.view(-1) == ref_tok[:, i]) | near_tie_ok(ref_logits[i], t.view(-1))
        assert bool(ok.all()), (i, t.view(-1), ref_tok[:, i])
    # the KV cache after prefill + one step is what the oracle holds, bit for bit in all but a sliver of slots
    # (k depends on the wqkv GEMM's summation order): compare through the tolerance of the tensor
    caches_ref = O.setup_caches(ocfg, 1, T + 2, BF, DEV)
    O.forward_ladder(ocfg, P, caches_ref, rows[:1], torch.arange(T, device=DEV))
    for layer in (0, 15, 31):
        kc = model.layers[layer].attention.kv_cache.k_cache[:1, :, :T]
        assert rel_err(kc, caches_ref.k[layer][:1, :, :T]) <= REL_TOL, layer


def test_ladder_405b_tp8_shard_config5_full():
    """Config 5: one TP=8 rank shard of Ladder-405B (dim 16384, 126 layers, 16 q / 1 kv heads per rank,
    FFN 6656, Llama-3.1 RoPE scaling, ~101 GB of weights), batch 16, context 4096, 64 new tokens."""
    progress("cfg5: building (101 GB of weights)")
    stats = run_parity(build("ladder", **shape_kw("ladder-405b-tp8")), "ladder", B=16, T=4096, new=64)
    report("cfg5 ladder-405b-tp8 B=16", stats)
    check(stats)
    torch.cuda.empty_cache()
