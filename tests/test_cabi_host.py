"""CPU-side checks of the C-ABI library and the host logic above it (no kernel is launched).

* libladder_hip.so loads and exports every symbol include/ladder_hip.h declares, and the ctypes
  prototypes of gpt_fast/_hip.py cover exactly that set;
* argument validation answers before anything touches the device;
* the configuration registry reproduces the reference's shapes (gpt_ladder_TP.py:20-207) and the
  per-rank sizes of the benchmark configurations;
* modules built on the meta device carry the reference's parameter names and shapes;
* bytes-per-step accounting used for the roofline."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ladder_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lr_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from gpt_fast import _hip

    if not os.path.exists(_hip.lib_path()):
        pytest.fail(f"{_hip.lib_path()} has not been built (python ladder-residual-inference_amd/build.py)")
    return _hip.load()


def test_library_exports_every_declared_symbol(lib):
    from gpt_fast import _hip

    names = declared_symbols()
    assert len(names) >= 20
    raw = ctypes.CDLL(_hip.lib_path())
    missing = [n for n in names if not hasattr(raw, n)]
    assert not missing, missing
    assert sorted(_hip.exported_names()) == names


def test_version_and_error_strings(lib):
    assert lib.lr_version() >= 1
    seen = set()
    for code in range(0, -7, -1):
        s = lib.lr_error_string(code)
        assert s and s.decode()
        seen.add(s)
    assert len(seen) >= 6, "every error code has its own message"


def test_validation_precedes_any_device_work(lib):
    # null / misaligned pointers and impossible shapes are refused on the host (no GPU here)
    E_NULL, E_ALIGN, E_SHAPE = -1, -2, -3
    assert lib.lr_add(None, None, 1.0, None, 16, None) == E_NULL
    assert lib.lr_add(8, 16, 1.0, 32, 16, None) == E_ALIGN
    assert lib.lr_linear(None, 0, None, None, 0, 1, 8, 8, 0, None) == E_NULL
    assert lib.lr_linear(64, 8, 128, 256, 8, 0, 8, 8, 0, None) == E_SHAPE
    assert lib.lr_argmax(None, 0, None, 1, 8, None) == E_NULL
    from gpt_fast._hip import _Projection, EPI_SWIGLU
    import ctypes
    one = (_Projection * 1)(_Projection(64, 8, 128, 256, 8, 8, 8, 0))
    ptr = ctypes.cast(one, ctypes.c_void_p)
    assert lib.lr_linear_multi(None, 1, 1, None) == E_NULL
    assert lib.lr_linear_multi(ptr, 3, 1, None) == E_SHAPE          # at most two projections
    assert lib.lr_linear_multi(ptr, 1, 65, None) == -4              # more than 64 rows: unsupported
    one[0].epilogue = EPI_SWIGLU
    one[0].N = 7                                                    # [up; gate] rows come in pairs
    assert lib.lr_linear_multi(ptr, 1, 1, None) == E_SHAPE
    one[0].N, one[0].K = 8, 12                                      # K % 8
    assert lib.lr_linear_multi(ptr, 1, 1, None) == E_SHAPE          # ldx < K
    one[0].ldx = 16
    assert lib.lr_linear_multi(ptr, 1, 1, None) == E_ALIGN
    # attention beside a projection: attention arguments as lr_attn_decode, then what it has no kernel for
    one[0] = _Projection(64, 8, 128, 256, 8, 8, 8, 0)

    def beside(q, proj, M, epi=0, scratch_bytes=1 << 30):
        one[0].epilogue = epi
        return lib.lr_attn_decode_beside(q, 1024, 128, 256, 512, 1024, 1024, 4, 8, 1, 128, 64, 2048, scratch_bytes,
                                         proj, M, None)

    assert beside(None, ptr, 4) == E_NULL
    assert beside(64, None, 4) == E_NULL
    assert beside(64, ptr, 0) == E_SHAPE
    assert beside(64, ptr, 17) == -4                                # the 16-row band only
    assert beside(64, ptr, 4, epi=2) == -4                          # a projection that writes the cache
    assert beside(64, ptr, 4, scratch_bytes=16) == E_SHAPE
    # the prefill's q/k/v projection with the rotation and the cache writes in its output pass
    from gpt_fast._hip import _RopeKv
    rope = _RopeKv(64, 128, 192, 256, None, 8, 1, 128, 64, 64)          # N = (8 + 2) * 128 = 1280

    def fused(x=64, ldx=64, ldy=1280, M=8, K=64, S=4, r=rope):
        return lib.lr_linear_rope_kv(x, ldx, 128, 256, ldy, M, K, S, None if r is None else ctypes.byref(r), None)

    assert fused(x=None) == E_NULL
    assert fused(r=None) == E_NULL
    assert fused(M=9) == E_SHAPE                                        # whole sequences of S tokens
    assert fused(ldy=1272) == E_SHAPE                                   # ldy < N
    assert fused(ldy=1284) == E_ALIGN
    assert fused(K=60, ldx=64) == E_ALIGN
    assert fused(r=_RopeKv(64, None, 192, 256, None, 8, 1, 128, 64, 64)) == E_NULL      # no positions
    assert fused(r=_RopeKv(64, 128, 192, 256, None, 8, 1, 124, 64, 64), ldy=1240) == E_ALIGN   # head_dim % 8
    from gpt_fast._hip import _ProjectionFp8
    one8 = (_ProjectionFp8 * 1)(_ProjectionFp8(64, 16, 128, 192, 256, 8, 8, 16, 0))
    ptr8 = ctypes.cast(one8, ctypes.c_void_p)
    assert lib.lr_linear_fp8_multi(None, 1, 1, None) == E_NULL
    assert lib.lr_linear_fp8_multi(ptr8, 1, 17, None) == -4           # up to 16 rows
    assert lib.lr_linear_fp8_multi(ptr8, 3, 1, None) == E_SHAPE
    one8[0].K = 24                                                    # 16 weights per lane and load
    assert lib.lr_linear_fp8_multi(ptr8, 1, 1, None) == E_SHAPE       # ldx < K
    one8[0].ldx = 24
    assert lib.lr_linear_fp8_multi(ptr8, 1, 1, None) == E_ALIGN
    one8[0].K, one8[0].ldx, one8[0].scales = 16, 16, None
    assert lib.lr_linear_fp8_multi(ptr8, 1, 1, None) == E_NULL
    assert lib.lr_ladder_decode_step(None, 1, None, None, None, 0, None, 0, None, None, 0, 0, 0, None, 0, None) == E_NULL
    assert lib.lr_ladder_decode_step_fp8(None, 1, None, None, None, 0, None, 0, None, None, 0, 0, 0, None, 0, None) == E_NULL
    assert lib.lr_ladder_step_workspace_bytes(None, 1) == 0


def test_missing_library_is_an_error(monkeypatch):
    from gpt_fast import _hip

    monkeypatch.setattr(_hip, "_lib", None)
    monkeypatch.setattr(_hip, "_LIB_PATH", os.path.join(ROOT, "no_such_dir", "libladder_hip.so"))
    with pytest.raises(_hip.LadderHipError):
        _hip.load()


def test_registry_matches_reference_shapes():
    from gpt_fast.config import ModelArgs, args_from_name

    a = args_from_name("ladder", "llama-3-8b")
    assert (a.dim, a.n_layer, a.n_head, a.n_local_heads, a.intermediate_size, a.vocab_size) == \
        (4096, 32, 32, 8, 14336, 128256)
    assert a.head_dim == 128 and a.rope_base == 500000
    # default intermediate size: round_up(int(8 * dim / 3), 256)   (gpt_ladder_TP.py:56-60)
    b = ModelArgs(dim=1000, n_head=8, n_layer=1)
    assert b.intermediate_size == 2816 and b.n_local_heads == 8 and b.head_dim == 125
    # one tensor-parallel rank of Ladder-70B at TP = 8
    c = args_from_name("ladder", "ladder-70b-tp8")
    assert (c.tp_world_size, c.n_head_local, c.n_kv_local, c.ffn_local, c.output_rows) == (8, 8, 1, 3584, 16032)
    d = args_from_name("ladder", "ladder-405b-tp8")
    assert (d.dim, d.n_layer, d.n_head_local, d.n_kv_local, d.ffn_local) == (16384, 126, 16, 1, 6656)
    with pytest.raises(AssertionError):
        ModelArgs(dim=512, n_head=8, n_layer=1, intermediate_size=1022, tp_world_size=4)   # not divisible by tp
    from gpt_fast.utils import Attention

    with pytest.raises(AssertionError), torch.device("meta"):   # heads not divisible by tp (utils.py:155-162)
        Attention(ModelArgs(dim=512, n_head=8, n_local_heads=2, n_layer=1, intermediate_size=1024, tp_world_size=4))


@pytest.mark.parametrize("family", ["ladder", "dense", "desync", "parallel"])
def test_meta_modules_have_reference_parameter_names(family):
    import benchmark as bm
    from gpt_fast.config import ModelArgs
    from oracle import ladder_oracle as O

    kw = dict(block_size=64, vocab_size=512, n_layer=2, n_head=4, n_local_heads=2, dim=256, intermediate_size=512)
    cls = {"ladder": bm.GPTLadder, "dense": bm.GPTDense, "desync": bm.GPTDesync, "parallel": bm.GPTParallel}[family]
    with torch.device("meta"):
        model = cls(ModelArgs(**kw))
    got = {n: tuple(p.shape) for n, p in model.named_parameters()}
    want = dict(O.param_shapes(O.OracleConfig(**kw), family))
    assert got == want


def test_virtual_tp_builds_one_rank_without_a_process_group(monkeypatch):
    from gpt_fast import maybe_init_dist, tp

    assert maybe_init_dist() == 0
    tp.set_virtual_tp(8, 3)
    try:
        assert tp.get_tp_world_size() == 8 and tp.get_tp_rank() == 3
    finally:
        tp.set_virtual_tp(1, 0)
    with pytest.raises(AssertionError):
        tp.set_virtual_tp(4, 4)
    assert not torch.distributed.is_initialized()
    monkeypatch.setenv("WORLD_SIZE", "2")     # a multi-process launch is refused, never silently run
    with pytest.raises(RuntimeError):
        maybe_init_dist()


def test_shard_vocab_flag_reaches_the_model_shape():
    """benchmark.py --virtual_tp N --shard_vocab: the lm_head of the unsharded registry names is built at
    vocab_size / N rows (the reference's flag surface is benchmark.py:498-518; it replicates the head)."""
    import benchmark as bm
    from gpt_fast import tp
    from gpt_fast.config import args_from_name

    args = bm.build_parser().parse_args(["--model_name", "gpt_ladder:70B", "--prompt_length", "8", "--virtual_tp", "8",
                                         "--shard_vocab"])
    assert args.shard_vocab and args.virtual_tp == 8
    tp.set_virtual_tp(args.virtual_tp, args.tp_rank, args.shard_vocab)
    try:
        c = args_from_name("ladder", "70B")
        assert c.tp_world_size == 8 and c.shard_vocab and c.output_rows == c.vocab_size // 8
        assert c.n_head_local == 8 and c.n_kv_local == 1 and c.ffn_local == 3584
    finally:
        tp.set_virtual_tp(1, 0)
    c = args_from_name("ladder", "70B")
    assert not c.shard_vocab and c.output_rows == c.vocab_size
    assert not bm.build_parser().parse_args(["--model_name", "gpt_ladder:70B", "--prompt_length", "8"]).shard_vocab


def test_bytes_per_step_accounting():
    import benchmark as bm
    from gpt_fast.config import args_from_name

    c = args_from_name("ladder", "ladder-70b-tp8")
    b0 = bm.decode_bytes_per_step(c, 1, 2048)
    # weights 17.378 GB + valid KV + KV write + embedding row + logits: 17.462 GB at position 2048
    assert abs(b0 - 17.462e9) < 0.003e9
    # one more position costs one more K and V row per layer
    assert bm.decode_bytes_per_step(c, 1, 2049) - b0 == 80 * 2 * 128 * 2
    # a second sequence adds its KV, embedding row and logits, not the weights
    assert bm.decode_bytes_per_step(c, 2, 2048) - b0 < 0.1e9


def _desc(**over):
    from gpt_fast import _hip

    kw = dict(dim=256, n_layer=2, n_head=4, n_kv_head=2, head_dim=64, ffn=512, out_rows=512, vocab=512, smax=64,
              block_size=64, eps=1e-5, attention_workgroups=0, tok_embeddings=4096, norm=4096, output=4096,
              freqs_cis=4096, layers_dev=4096)
    kw.update(over)
    return _hip.LadderModelDesc(**kw)


def test_step_descriptor_is_validated_on_the_host(lib):
    """Shapes the one-kernel step must refuse are refused before any device is looked at (no GPU here)."""
    import ctypes

    E_NULL, E_SHAPE, E_UNSUPPORTED = -1, -3, -4
    # (the workspace pointer is misaligned on purpose: where a GPU is present a descriptor that passes validation is
    # then refused with LR_E_ALIGN instead of being initialised at a made-up address)
    init = lambda d, b=1: lib.lr_ladder_step_init(ctypes.byref(d), b, 8, 1 << 20, None)
    # a cache longer than the RoPE table: positions beyond block_size would read past the end of freqs_cis
    assert init(_desc(smax=72, block_size=64)) == E_SHAPE
    assert lib.lr_ladder_step_workspace_bytes(ctypes.byref(_desc(smax=72, block_size=64)), 1) == 0
    assert init(_desc(smax=64, block_size=60)) != E_SHAPE          # the cache length is rounded up to 8
    assert init(_desc(n_head=5)) == E_SHAPE                        # q heads not a multiple of kv heads
    assert init(_desc(), b=3) == E_UNSUPPORTED                     # batch: 1 or 2
    assert init(_desc(head_dim=48)) == E_UNSUPPORTED
    assert init(_desc(dim=20000)) == E_UNSUPPORTED


def test_load_hook_fuses_separate_projections():
    """utils.py:178-185: checkpoints with wq / wk / wv load into the fused wqkv, rows [q; k; v]."""
    from gpt_fast.config import ModelArgs
    from gpt_fast.utils import Attention

    cfg = ModelArgs(dim=64, n_head=4, n_local_heads=2, n_layer=1, intermediate_size=128)
    att = Attention(cfg)
    g = torch.Generator().manual_seed(0)
    wq, wk, wv = (torch.randn(r, 64, generator=g) for r in (64, 32, 32))
    wo = torch.randn(64, 64, generator=g)
    att.load_state_dict({"wq.weight": wq, "wk.weight": wk, "wv.weight": wv, "wo.weight": wo})
    assert torch.equal(att.wqkv.weight, torch.cat([wq, wk, wv])) and torch.equal(att.wo.weight, wo)
    # an already fused checkpoint passes through untouched
    att2 = Attention(cfg)
    att2.load_state_dict(att.state_dict())
    assert torch.equal(att2.wqkv.weight, att.wqkv.weight)


def test_setup_caches_refuses_a_sequence_longer_than_block_size():
    import benchmark as bm
    from gpt_fast.config import ModelArgs

    with torch.device("meta"):
        model = bm.GPTLadder(ModelArgs(block_size=64, vocab_size=512, n_layer=1, n_head=4, dim=256))
    with pytest.raises(ValueError):
        model.setup_caches(1, 65)
