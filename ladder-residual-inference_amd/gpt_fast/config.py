"""Hyper-parameters and the name -> shape registry, one copy for all four block families.

The reference keeps four diverging copies of ModelArgs / transformer_configs
(gpt_ladder_TP.py:32-207, gpt_dense_TP.py:29-181, gpt_desync_TP.py:30-248,
gpt_parallel_TP.py:29-131).  Here one shape table is shared and each family lists the names it
exposes plus its own extras (the desync reduce patterns, the semi-compiled aliases, desync's
36-head "3b").  Added on top: an explicit tensor-parallel world size that is NOT tied to
torch.distributed (a rank shard can be built in a single process), an optional vocab-sharded
lm_head, and the benchmark shapes "ladder-1b", "ladder-8b", "ladder-70b-tp8", "ladder-405b-tp8"."""
from dataclasses import dataclass
from typing import Dict, List, Optional

from . import tp as _tp


def find_multiple(n: int, k: int) -> int:
    return n if n % k == 0 else n + k - (n % k)


@dataclass
class ModelArgs:
    block_size: int = 2048
    vocab_size: int = 32000
    n_layer: int = 32
    n_head: int = 32
    dim: int = 4096
    intermediate_size: Optional[int] = None
    n_local_heads: int = -1
    head_dim: int = 64
    rope_base: float = 10000
    norm_eps: float = 1e-5
    rope_scaling: Optional[dict] = None
    semi_compiled_model: bool = False
    # desync family (gpt_desync_TP.py:44-45)
    reduce_pattern: Optional[List[Dict[str, bool]]] = None
    force_disable_last_all_reduce: bool = False
    # ladder family: the layers that run the ladder schedule (None: all of them, as gpt_ladder_TP.py does; a list
    # is the partial-ladder wiring of hf_modeling_utils/modeling_llama_ladder.py:889-948: the others are dense)
    ladder_layers: Optional[List[int]] = None
    # rank shard: None -> the process-wide virtual setting of gpt_fast.tp
    tp_world_size: Optional[int] = None
    tp_rank: Optional[int] = None
    # lm_head keeps vocab_size // tp_world_size rows (the reference replicates the full head); None -> the
    # process-wide virtual setting of gpt_fast.tp
    shard_vocab: Optional[bool] = None

    def __post_init__(self):
        if self.tp_world_size is None:
            self.tp_world_size = _tp.get_tp_world_size()
        if self.tp_rank is None:
            self.tp_rank = _tp.get_tp_rank() if self.tp_world_size == _tp.get_tp_world_size() else 0
        if self.shard_vocab is None:
            self.shard_vocab = _tp.get_shard_vocab() if self.tp_world_size == _tp.get_tp_world_size() else False
        if self.n_local_heads == -1:
            self.n_local_heads = self.n_head
        if self.intermediate_size is None:
            self.intermediate_size = find_multiple(int(2 * (4 * self.dim) / 3), 256)
        self.head_dim = self.dim // self.n_head
        tp = self.tp_world_size
        assert self.dim % tp == 0
        assert self.intermediate_size % tp == 0
        if self.reduce_pattern is None:
            self.reduce_pattern = [{"attention": False, "mlp": True} for _ in range(self.n_layer)]
        if self.ladder_layers is not None:
            assert all(0 <= i < self.n_layer for i in self.ladder_layers)
            if sorted(self.ladder_layers) == list(range(self.n_layer)):
                self.ladder_layers = None

    def is_ladder_layer(self, i: int) -> bool:
        return self.ladder_layers is None or i in self.ladder_layers

    # per-rank sizes
    @property
    def n_head_local(self) -> int:
        return self.n_head // self.tp_world_size

    @property
    def n_kv_local(self) -> int:
        return self.n_local_heads // self.tp_world_size

    @property
    def ffn_local(self) -> int:
        return self.intermediate_size // self.tp_world_size

    @property
    def output_rows(self) -> int:
        if self.shard_vocab:
            assert self.vocab_size % self.tp_world_size == 0
            return self.vocab_size // self.tp_world_size
        return self.vocab_size


# name: (block_size, vocab, layers, q heads, kv heads or None (= q heads), dim, ffn or None (= default), rope base)
_SHAPES = {
    "CodeLlama-7b-Python-hf": (16384, 32000, 32, 32, None, 4096, None, 1000000),
    "1b": (2048, 49152, 40, 24, 24, 1536, 4096, 10000),
    "1.55b": (2048, 49152, 52, 24, 24, 1536, 4096, 10000),
    "3b": (2048, 49152, 40, 32, 32, 2304, 9216, 10000),
    "3b-36h": (2048, 49152, 40, 36, 36, 2304, 9216, 10000),
    "3.9bh": (2048, 49152, 52, 32, 32, 2304, 9216, 10000),
    "3.9bw1": (2048, 49152, 40, 32, 32, 3200, 9216, 10000),
    "3.9bw2": (2048, 49152, 40, 32, 32, 2560, 11000, 10000),
    "7B": (2048, 32000, 32, 32, None, 4096, None, 10000),
    "13B": (2048, 32000, 40, 40, None, 5120, None, 10000),
    "30B": (2048, 32000, 60, 52, None, 6656, None, 10000),
    "34B": (2048, 32000, 48, 64, 8, 8192, 22016, 1000000),
    "70B": (2048, 32000, 80, 64, 8, 8192, 28672, 10000),
    "Mistral-7B": (2048, 32000, 32, 32, 8, 4096, 14336, 10000),
    "stories15M": (2048, 32000, 6, 6, None, 288, None, 10000),
    "stories110M": (2048, 32000, 12, 12, None, 768, None, 10000),
    "llama-3.2-1b": (2048, 128256, 16, 32, None, 2048, 8192, 10000),
    "llama-3.2-3b": (2048, 128256, 28, 24, None, 3072, 8192, 10000),
    "llama-3-8b-4layers": (8192, 128256, 4, 32, 8, 4096, 14336, 500000),
    "llama-3-8b": (8192, 128256, 32, 32, 8, 4096, 14336, 500000),
    "llama-3-70b": (8192, 128256, 80, 64, 8, 8192, 28672, 500000),
    "llama-3.1-405b": (131072, 128256, 126, 128, 16, 16384, 53248, 500000),
    "bloom-176b": (8192, 250880, 70, 112, 112, 14336, 50176, 500000),
    # benchmark shapes of this build (global sizes; the -tp8 ones are built as rank shards)
    "ladder-1b": (2048, 128256, 16, 32, 8, 2048, 8192, 500000),
    "ladder-8b": (8192, 128256, 32, 32, 8, 4096, 14336, 500000),
    "ladder-70b-tp8": (8192, 128256, 80, 64, 8, 8192, 28672, 500000),
    "ladder-405b-tp8": (131072, 128256, 126, 128, 8, 16384, 53248, 500000),
}
_LLAMA31_SCALING = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)
_EXTRA = {
    "llama-3.1-405b": dict(rope_scaling=_LLAMA31_SCALING),
    "ladder-70b-tp8": dict(tp_world_size=8, tp_rank=0, shard_vocab=True),
    "ladder-405b-tp8": dict(rope_scaling=_LLAMA31_SCALING, tp_world_size=8, tp_rank=0, shard_vocab=True),
}
_BENCH = ["ladder-1b", "ladder-8b", "ladder-70b-tp8", "ladder-405b-tp8"]
_COMMON = ["CodeLlama-7b-Python-hf", "1b", "3b", "7B", "13B", "30B", "34B", "70B", "Mistral-7B", "stories15M",
           "stories110M", "llama-3-8b", "llama-3-70b", "llama-3.1-405b"]


def _shape(name: str, **over) -> dict:
    bs, vocab, nl, nh, nkv, dim, ffn, base = _SHAPES[name]
    d = dict(block_size=bs, vocab_size=vocab, n_layer=nl, n_head=nh, dim=dim, rope_base=base)
    if nkv is not None:
        d["n_local_heads"] = nkv
    if ffn is not None:
        d["intermediate_size"] = ffn
    d.update(_EXTRA.get(name, {}))
    d.update(over)
    return d


def _never(n):
    return [{"attention": False, "mlp": False} for _ in range(n)]


def _every_other(n):
    return [{"attention": False, "mlp": False}, {"attention": False, "mlp": True}] * (n // 2)


def _build_family(family: str) -> Dict[str, dict]:
    names = list(_COMMON) + _BENCH
    reg: Dict[str, dict] = {}
    if family in ("ladder", "dense", "parallel"):
        names += ["llama-3.2-1b", "llama-3.2-3b"]
        reg["70B-semi-compiled"] = _shape("70B", semi_compiled_model=True)
    if family in ("ladder", "dense"):
        names += ["3.9bh", "3.9bw1", "3.9bw2", "bloom-176b"]
    if family == "ladder":
        names += ["1.55b"]
        reg["llama-3-8b-semi-compiled"] = _shape("llama-3-8b", semi_compiled_model=True)
        reg["llama-3-70b-semi-compiled"] = _shape("llama-3-70b", semi_compiled_model=True)
    if family == "dense":
        names += ["llama-3-8b-4layers"]
    for n in names:
        reg[n] = _shape(n)
    if family == "desync":
        # gpt_desync_TP.py:79-113: "1b" itself never reduces, "1b-upper-bound" is the default pattern;
        # "3b" has 36 heads in this family only.
        reg["1b"] = _shape("1b", reduce_pattern=_never(40), force_disable_last_all_reduce=True)
        reg["1b-upper-bound"] = _shape("1b")
        reg["3b"] = _shape("3b-36h")
        reg["3b-upper-bound"] = _shape("3b-36h", reduce_pattern=_never(40), force_disable_last_all_reduce=True)
        reg["70B-infinite"] = _shape("70B", reduce_pattern=_never(80))
        reg["70B-semi-compiled"] = _shape("70B", semi_compiled_model=True)
        reg["70B-infinite-semi-compiled"] = _shape("70B", semi_compiled_model=True, reduce_pattern=_never(80))
        for base, n in (("llama-3-8b", 32), ("llama-3-70b", 80)):
            reg[base + "-4x"] = _shape(base, reduce_pattern=_every_other(n))
            reg[base + "-upper-bound"] = _shape(base, reduce_pattern=_never(n), force_disable_last_all_reduce=True)
        reg["llama-3-8b-infinite"] = _shape("llama-3-8b", reduce_pattern=_never(32))
        reg["llama-3.1-405b-upper-bound"] = _shape("llama-3.1-405b", reduce_pattern=_never(126),
                                                   force_disable_last_all_reduce=True)
        for n in _BENCH:  # the no-communication schedule on the benchmark shapes
            reg[n + "-upper-bound"] = _shape(n, reduce_pattern=_never(_SHAPES[n][2]),
                                             force_disable_last_all_reduce=True)
    return reg


REGISTRIES = {f: _build_family(f) for f in ("ladder", "dense", "desync", "parallel")}


def args_from_name(family: str, name: str) -> ModelArgs:
    reg = REGISTRIES[family]
    if name not in reg:
        # the reference returns None here and fails later with an AttributeError (gpt_ladder_TP.py:59-62)
        raise KeyError(f"unknown {family} config '{name}'; known: {sorted(reg)}")
    return ModelArgs(**reg[name])
