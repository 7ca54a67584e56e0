"""Loading real checkpoints into one tensor-parallel rank of the HIP models.

Three steps, each usable on its own (all on plain state dicts, CPU tensors are fine):

  convert_hf_state_dict   Hugging Face Llama / Llama-Ladder names (hf_modeling_utils/
                          modeling_llama_ladder.py: `model.layers.N.self_attn.{q,k,v,o}_proj`,
                          `mlp.{gate,up,down}_proj`, `input_layernorm`, `post_attention_layernorm`,
                          `model.embed_tokens`, `model.norm`, `lm_head`) -> the reference's gpt_fast
                          names with fused projections: `attention.wqkv` rows [q; k; v]
                          (utils.py:191), `feed_forward.w1` rows [up; gate] (utils.py:145-148).
                          The rows of q and k are re-ordered per head from the half-split RoPE
                          layout of the HF model (rotate_half, modeling_llama_ladder.py:195-226) to
                          the interleaved pairs gpt_fast rotates (utils.py:120-132).
  shard_state_dict        the slice of an UN-SHARDED gpt_fast state dict that rank r of tp owns,
                          exactly as the reference's layers are sized (utils.py:142-143, 165-176):
                          wqkv -> [q_r; k_r; v_r], w1 -> [u_r; g_r], wo[:, r], w2[:, r], norms and
                          the embedding table replicated, lm_head rows r (only with shard_vocab).
                          Separate wq / wk / wv (utils.py:178-185) are accepted and fused.
  load_checkpoint         convert if needed, shard, cast, and load into a GPT* module.

`model_args_from_hf_config` turns the fields of an HF config.json (hf_modeling_utils/configs/*.json)
into ModelArgs keywords, `ladder_layers` included (configuration_llama_ladder.py:32-45)."""
import json
import os
from typing import Dict, List, Optional, Union

import torch
from torch import Tensor

StateDict = Dict[str, Tensor]


# ------------------------------------------------------------------------------------------------
# Hugging Face names -> gpt_fast names
# ------------------------------------------------------------------------------------------------

def _interleave_rope_rows(w: Tensor, n_head: int) -> Tensor:
    """Rows of a q or k projection [n_head * hd, dim]: within each head, HF keeps the rotation pair
    (j, j + hd/2); gpt_fast rotates the pair (2j, 2j + 1).  New row 2j <- old row j, new row
    2j + 1 <- old row j + hd/2."""
    rows, dim = w.shape
    hd = rows // n_head
    return w.view(n_head, 2, hd // 2, dim).transpose(1, 2).reshape(rows, dim)


def is_hf_state_dict(sd: StateDict) -> bool:
    return any(k.startswith("model.layers.") or k == "model.embed_tokens.weight" for k in sd)


def convert_hf_state_dict(sd: StateDict, n_head: int, n_kv_head: int, head_dim: Optional[int] = None) -> StateDict:
    """HF Llama(-Ladder) state dict -> gpt_fast state dict (fused projections).  n_head / n_kv_head are the head
    counts of the tensors AS GIVEN: the global ones for an un-sharded checkpoint, the per-rank ones for a slice.
    With head_dim the q / k row counts are checked against them (a wrong head count would permute rows silently)."""
    out: StateDict = {}
    layers = sorted({int(k.split(".")[2]) for k in sd if k.startswith("model.layers.")})
    out["tok_embeddings.weight"] = sd["model.embed_tokens.weight"]
    for i in layers:
        src, dst = f"model.layers.{i}.", f"layers.{i}."
        if head_dim is not None:
            for name, heads in (("q_proj", n_head), ("k_proj", n_kv_head)):
                rows = sd[src + f"self_attn.{name}.weight"].shape[0]
                if rows != heads * head_dim:
                    raise ValueError(f"{src}self_attn.{name}.weight has {rows} rows, expected {heads} heads x {head_dim}")
        q = _interleave_rope_rows(sd[src + "self_attn.q_proj.weight"], n_head)
        k = _interleave_rope_rows(sd[src + "self_attn.k_proj.weight"], n_kv_head)
        v = sd[src + "self_attn.v_proj.weight"]
        out[dst + "attention.wqkv.weight"] = torch.cat([q, k, v])
        out[dst + "attention.wo.weight"] = sd[src + "self_attn.o_proj.weight"]
        out[dst + "feed_forward.w1.weight"] = torch.cat([sd[src + "mlp.up_proj.weight"], sd[src + "mlp.gate_proj.weight"]])
        out[dst + "feed_forward.w2.weight"] = sd[src + "mlp.down_proj.weight"]
        out[dst + "attention_norm.weight"] = sd[src + "input_layernorm.weight"]
        out[dst + "ffn_norm.weight"] = sd[src + "post_attention_layernorm.weight"]
    out["norm.weight"] = sd["model.norm.weight"]
    # tie_word_embeddings checkpoints carry no lm_head
    out["output.weight"] = sd.get("lm_head.weight", sd["model.embed_tokens.weight"])
    return out


def model_args_from_hf_config(cfg: Union[str, dict], **overrides) -> dict:
    """ModelArgs keywords from an HF config.json (path or parsed dict)."""
    if isinstance(cfg, (str, os.PathLike)):
        with open(cfg) as f:
            cfg = json.load(f)
    n_layer = cfg["num_hidden_layers"]
    kw = dict(block_size=cfg.get("max_position_embeddings", 2048), vocab_size=cfg["vocab_size"], n_layer=n_layer,
              n_head=cfg["num_attention_heads"], n_local_heads=cfg.get("num_key_value_heads", cfg["num_attention_heads"]),
              dim=cfg["hidden_size"], intermediate_size=cfg["intermediate_size"],
              rope_base=cfg.get("rope_theta", 10000.0), norm_eps=cfg.get("rms_norm_eps", 1e-5))
    scaling = cfg.get("rope_scaling")
    if scaling:
        kind = scaling.get("rope_type", scaling.get("type"))
        if kind != "llama3":
            raise ValueError(f"rope_scaling of type {kind!r} is not supported (the reference implements llama3 only)")
        kw["rope_scaling"] = {k: scaling[k] for k in ("factor", "low_freq_factor", "high_freq_factor",
                                                      "original_max_position_embeddings")}
    # configuration_llama_ladder.py:38-45: no field (a plain Llama config.json) or null means NO ladder layer -- every
    # block dense -- and an int means "the last n layers".  (ModelArgs itself reads None as "all layers", the
    # gpt_fast convention, so the absent field must not be passed on as None.)
    ladder = cfg.get("ladder_layers")
    if ladder is None:
        kw["ladder_layers"] = []
    elif isinstance(ladder, int):
        kw["ladder_layers"] = list(range(n_layer - ladder, n_layer))
    elif isinstance(ladder, list):
        kw["ladder_layers"] = list(ladder)
    else:
        raise ValueError(f"Invalid ladder_layers type: {type(ladder)}")
    kw.update(overrides)
    return kw


# ------------------------------------------------------------------------------------------------
# one rank's slice of an un-sharded gpt_fast state dict
# ------------------------------------------------------------------------------------------------

def _rows(w: Tensor, rank: int, tp: int) -> Tensor:
    n = w.shape[0]
    assert n % tp == 0, (tuple(w.shape), tp)
    return w[rank * (n // tp):(rank + 1) * (n // tp)]


def _cols(w: Tensor, rank: int, tp: int) -> Tensor:
    n = w.shape[1]
    assert n % tp == 0, (tuple(w.shape), tp)
    return w[:, rank * (n // tp):(rank + 1) * (n // tp)]


def shard_state_dict(sd: StateDict, n_head: int, n_kv_head: int, head_dim: int, tp: int, rank: int,
                     shard_vocab: bool = False) -> StateDict:
    """Rank `rank` of `tp` of an un-sharded state dict in the reference's names.  Handles the
    standard blocks (attention.wqkv / wq,wk,wv, attention.wo, feed_forward.w1, feed_forward.w2) and
    the parallel block's attention.wqkv1 ([q; k; v; up; gate]) and attention.w2."""
    assert 0 <= rank < tp and n_head % tp == 0 and n_kv_head % tp == 0
    nq, nkv = n_head * head_dim, n_kv_head * head_dim
    sd = dict(sd)
    # separate projections first become the fused matrix (utils.py:178-185)
    for key in [k for k in sd if k.endswith("attention.wq.weight")]:
        pre = key[: -len("wq.weight")]
        sd[pre + "wqkv.weight"] = torch.cat([sd.pop(pre + "wq.weight"), sd.pop(pre + "wk.weight"),
                                             sd.pop(pre + "wv.weight")])
    out: StateDict = {}
    for key, w in sd.items():
        if key.endswith("attention.wqkv.weight"):
            assert w.shape[0] == nq + 2 * nkv, (key, tuple(w.shape))
            q, k, v = w.split([nq, nkv, nkv])
            out[key] = torch.cat([_rows(q, rank, tp), _rows(k, rank, tp), _rows(v, rank, tp)])
        elif key.endswith("attention.wqkv1.weight"):
            ffn = (w.shape[0] - nq - 2 * nkv) // 2
            q, k, v, u, g = w.split([nq, nkv, nkv, ffn, ffn])
            out[key] = torch.cat([_rows(t, rank, tp) for t in (q, k, v, u, g)])
        elif key.endswith("feed_forward.w1.weight"):
            u, g = w.chunk(2)
            out[key] = torch.cat([_rows(u, rank, tp), _rows(g, rank, tp)])
        elif key.endswith(("attention.wo.weight", "feed_forward.w2.weight", "attention.w2.weight")):
            out[key] = _cols(w, rank, tp)
        elif key == "output.weight":
            out[key] = _rows(w, rank, tp) if shard_vocab else w
        else:   # norm gains, embedding table: every rank holds them whole
            out[key] = w
    return out


# ------------------------------------------------------------------------------------------------
# into a module
# ------------------------------------------------------------------------------------------------

def read_state_dict(path: str) -> StateDict:
    """A .safetensors file, a torch file (loaded with weights_only=True), or a directory of shards of
    either kind (every *.safetensors, else every *.bin / *.pt / *.pth)."""
    if os.path.isdir(path):
        names = sorted(os.listdir(path))
        files = [n for n in names if n.endswith(".safetensors")] or \
                [n for n in names if n.endswith((".bin", ".pt", ".pth"))]
        if not files:
            raise FileNotFoundError(f"no checkpoint files in {path}")
        sd: StateDict = {}
        for n in files:
            sd.update(read_state_dict(os.path.join(path, n)))
        return sd
    if path.endswith(".safetensors"):
        from safetensors.torch import load_file

        return load_file(path)
    try:
        sd = torch.load(path, map_location="cpu", weights_only=True, mmap=True)
    except (RuntimeError, ValueError):   # a legacy (non-zip) torch file cannot be memory-mapped
        sd = torch.load(path, map_location="cpu", weights_only=True)
    return sd.get("model", sd) if isinstance(sd, dict) and "model" in sd and isinstance(sd["model"], dict) else sd


def load_checkpoint(model: torch.nn.Module, checkpoint: Union[str, StateDict], already_sharded: bool = False) -> List[str]:
    """Load an un-sharded checkpoint (HF or gpt_fast names; a path or a state dict) into `model`,
    which was built for one tensor-parallel rank (model.config.tp_world_size / tp_rank).
    Returns the names of the tensors that were loaded.  Raises on missing or unexpected
    parameters; buffers the checkpoint does not carry (KV caches, masks) are left alone."""
    cfg = model.config
    sd = read_state_dict(checkpoint) if isinstance(checkpoint, (str, os.PathLike)) else dict(checkpoint)
    if is_hf_state_dict(sd):
        # an already sharded checkpoint holds this rank's heads only
        heads = (cfg.n_head_local, cfg.n_kv_local) if already_sharded else (cfg.n_head, cfg.n_local_heads)
        sd = convert_hf_state_dict(sd, heads[0], heads[1], cfg.head_dim)
    if not already_sharded:
        sd = shard_state_dict(sd, cfg.n_head, cfg.n_local_heads, cfg.head_dim, cfg.tp_world_size, cfg.tp_rank,
                              cfg.shard_vocab)
    if "attention.wqkv1.weight" in "".join(n for n, _ in model.named_parameters()) and \
            not any(k.endswith("wqkv1.weight") for k in sd):
        # the parallel block fuses the two projections and keeps the MLP's w2 under `attention`
        for key in [k for k in sd if k.endswith("attention.wqkv.weight")]:
            pre = key[: -len("attention.wqkv.weight")]
            sd[pre + "attention.wqkv1.weight"] = torch.cat([sd.pop(key), sd.pop(pre + "feed_forward.w1.weight")])
            sd[pre + "attention.w2.weight"] = sd.pop(pre + "feed_forward.w2.weight")
            sd.pop(pre + "ffn_norm.weight", None)
    params = dict(model.named_parameters())
    missing = sorted(set(params) - set(sd))
    unexpected = sorted(set(sd) - set(params))
    if missing or unexpected:
        raise KeyError(f"checkpoint does not match the model: missing {missing[:6]}, unexpected {unexpected[:6]}")
    with torch.no_grad():
        for name, p in params.items():
            w = sd[name]
            if tuple(w.shape) != tuple(p.shape):
                raise ValueError(f"{name}: checkpoint slice {tuple(w.shape)} vs parameter {tuple(p.shape)}")
            p.copy_(w.to(dtype=p.dtype))
    return sorted(params)
