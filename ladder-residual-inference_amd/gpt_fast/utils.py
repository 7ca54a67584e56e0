"""Per-rank building blocks shared by the four block families, on the gfx950 kernels.

Same classes, attribute names and call signatures as the reference's gpt_fast/utils.py
(KVCache :43-59, RMSNorm :62-78, precompute_freqs_cis :103-117, FeedForward :135-149,
Attention :152-260, FuseAttentionMLP :263-387, all_reduce_func :390-397, _get_model_size
:400-409), so state dicts and calling code carry over.  Every forward() enqueues HIP kernels of
libladder_hip.so on torch's current stream; nothing here computes with torch ops and there is no
CPU path.  The shard size comes from the config's (virtual) tensor-parallel world size and the
all-reduce is the identity: row-parallel outputs are this rank's partial sums."""
import itertools
import math
from contextlib import contextmanager
from typing import Optional

import torch
import torch.nn as nn
from torch import Tensor

from . import _hip

_USE_FLASH_ATTENTION: bool = False


@contextmanager
def set_flash_attention(enable: bool):
    """Kept for benchmark.py (--use_flash_attention).  The HIP attention kernels are the only
    attention path of this build, so the switch changes nothing."""
    global _USE_FLASH_ATTENTION
    previous, _USE_FLASH_ATTENTION = _USE_FLASH_ATTENTION, enable
    try:
        yield
    finally:
        _USE_FLASH_ATTENTION = previous


def is_flash_attention_enabled() -> bool:
    return _USE_FLASH_ATTENTION


class KVCache(nn.Module):
    """[max_batch, kv heads of this rank, max_seq, head_dim], zero-initialised (utils.py:43-59).  The model's own
    forward writes it in place from inside its projection kernels (lr_rope_kv_write and the RoPE + cache epilogues);
    update() is the reference's method for callers that hold the module themselves."""

    def __init__(self, max_batch_size, max_seq_length, n_heads, head_dim, dtype=torch.bfloat16):
        super().__init__()
        shape = (max_batch_size, n_heads, max_seq_length, head_dim)
        self.register_buffer("k_cache", torch.zeros(shape, dtype=dtype))
        self.register_buffer("v_cache", torch.zeros(shape, dtype=dtype))

    def update(self, input_pos: Tensor, k_val: Tensor, v_val: Tensor):
        """k_cache[:, :, input_pos] = k_val ([B, H, S, D]), the same for v; returns (k_cache, v_cache) as the
        reference does (utils.py:50-59).  One launch of lr_kv_update; positions stay on the device."""
        assert input_pos.shape[0] == k_val.shape[2]
        if k_val.stride(-1) != 1 or k_val.stride() != v_val.stride():
            k_val, v_val = k_val.contiguous(), v_val.contiguous()
        _hip.kv_update(k_val, v_val, input_pos.to(torch.int32), self.k_cache, self.v_cache)
        return self.k_cache, self.v_cache


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: Tensor) -> Tensor:
        x = x.contiguous()
        return _hip.add_rmsnorm(x, None, None, self.weight, None, torch.empty_like(x), self.eps)


def apply_rope_scaling(freqs: torch.Tensor, rope_scaling: dict) -> torch.Tensor:
    """Llama-3.1 frequency scaling: keep short wavelengths, divide long ones by `factor`, blend the
    band in between.  Same element-wise fp32 evaluation order as the reference (utils.py:81-100)."""
    factor = rope_scaling["factor"]
    low = rope_scaling["low_freq_factor"]
    high = rope_scaling["high_freq_factor"]
    old_len = rope_scaling["original_max_position_embeddings"]
    scaled = []
    for f in freqs:
        wavelen = 2 * math.pi / f
        if wavelen < old_len / high:
            scaled.append(f)
        elif wavelen > old_len / low:
            scaled.append(f / factor)
        else:
            t = (old_len / wavelen - low) / (high - low)
            scaled.append((1 - t) * f / factor + t * f)
    return torch.tensor(scaled, dtype=freqs.dtype)


def precompute_freqs_cis(seq_len: int, n_elem: int, base: int = 10000, dtype: torch.dtype = torch.bfloat16,
                         rope_scaling: Optional[dict] = None) -> Tensor:
    """(cos, sin) table [seq_len, n_elem/2, 2], evaluated in fp32 on the HOST (so its bits do not
    depend on the device) and then rounded to the model dtype."""
    with torch.device("cpu"):
        exponent = torch.arange(0, n_elem, 2)[: n_elem // 2].float() / n_elem
        freqs = 1.0 / (base ** exponent)
        if rope_scaling is not None:
            freqs = apply_rope_scaling(freqs, rope_scaling)
        angle = torch.outer(torch.arange(seq_len), freqs)
        table = torch.stack([angle.cos(), angle.sin()], dim=-1)
    return table.to(dtype=dtype)


def all_reduce_func(x: torch.Tensor, clone: bool, async_op=False):
    """The tensor-parallel SUM all-reduce of the reference, replaced by "keep the partial sum in
    this rank's buffer": returns the input and no handle."""
    return x, None


def _get_model_size(model):
    model_size = 0
    params = 0
    for _, child in model.named_children():
        if isinstance(child, torch.nn.Embedding):
            continue
        tensors = list(itertools.chain(child.parameters(), child.buffers()))
        model_size += sum(t.numel() * t.dtype.itemsize for t in tensors)
        params += sum(t.numel() for t in tensors)
    return model_size, params


def _pos_i32(input_pos: Tensor) -> Tensor:
    return input_pos if input_pos.dtype == torch.int32 else input_pos.to(torch.int32)


class FeedForward(nn.Module):
    """w1 rows are [up; gate] of this rank; w2 is row-parallel and returns a partial sum."""

    def __init__(self, config) -> None:
        super().__init__()
        tp = config.tp_world_size
        assert config.intermediate_size % tp == 0
        assert config.dim % tp == 0
        self.w1 = nn.Linear(config.dim, 2 * config.intermediate_size // tp, bias=False)
        self.w2 = nn.Linear(config.intermediate_size // tp, config.dim, bias=False)

    def forward(self, x: Tensor) -> Tensor:
        x = x.contiguous()
        lead = x.shape[:-1]
        h = _hip.module_linear(x, self.w1, x.new_empty(*lead, self.w1.out_features))
        return _hip.module_linear_swiglu(h, self.w2, x.new_empty(*lead, self.w2.out_features))


class _AttentionCore(nn.Module):
    """What Attention and FuseAttentionMLP share: head bookkeeping, RoPE + cache write, attention."""

    def _init_heads(self, config):
        tp = config.tp_world_size
        assert config.dim % config.n_head == 0
        assert config.dim % tp == 0
        assert config.n_head % tp == 0
        assert config.n_local_heads % tp == 0
        self.kv_cache = None
        self.head_dim = config.head_dim
        self.n_head = config.n_head // tp
        self.n_local_heads = config.n_local_heads // tp
        self.dim = config.dim // tp  # columns of wo on this rank (= n_head * head_dim when sharded)
        self._register_load_state_dict_pre_hook(self.load_hook)
        self._scratch = None

    def load_hook(self, state_dict, prefix, *args):
        """Checkpoints with separate wq / wk / wv are fused on load (reference utils.py:178-185)."""
        if prefix + "wq.weight" in state_dict:
            wq = state_dict.pop(prefix + "wq.weight")
            wk = state_dict.pop(prefix + "wk.weight")
            wv = state_dict.pop(prefix + "wv.weight")
            state_dict[prefix + "wqkv.weight"] = torch.cat([wq, wk, wv])

    def _attend(self, qkv: Tensor, bsz: int, seqlen: int, freqs_cis: Tensor, input_pos: Tensor) -> Tensor:
        """qkv [B, S, >= (Hq + 2 Hkv) hd] fresh from the fused projection -> y [B, S, Hq * hd]."""
        assert self.kv_cache is not None, "Caches must be initialized first"
        Hq, Hkv, hd = self.n_head, self.n_local_heads, self.head_dim
        pos = _pos_i32(input_pos)
        assert pos.shape[0] == seqlen
        kc, vc = self.kv_cache.k_cache, self.kv_cache.v_cache
        # module-level callers pass freqs_cis[input_pos] (one table row per token), as the reference does
        assert freqs_cis.shape[0] == seqlen
        _hip.rope_kv_write(qkv, freqs_cis.contiguous(), True, pos, kc, vc, bsz, seqlen, Hq, Hkv, hd)
        y = qkv.new_empty(bsz, seqlen, Hq * hd)
        if seqlen == 1:
            need = _hip.attn_decode_scratch_bytes(bsz, Hq, hd, kc.shape[2]) // 4
            if self._scratch is None or self._scratch.numel() < need or self._scratch.device != qkv.device:
                self._scratch = torch.empty(need, dtype=torch.float32, device=qkv.device)
            _hip.attn_decode(qkv, kc, vc, pos, y, self._scratch, bsz, Hq, Hkv, hd)
        else:
            _hip.attn_prefill(qkv, kc, vc, pos, y, bsz, seqlen, Hq, Hkv, hd)
        return y


class Attention(_AttentionCore):
    """wqkv rows are [q; k; v] of this rank; wo is row-parallel and returns a partial sum.
    `mask` is accepted for signature compatibility and not read: key j is visible to the query at
    position p iff j <= p, which is what the reference's causal_mask[input_pos] encodes."""

    def __init__(self, config):
        super().__init__()
        tp = config.tp_world_size
        total_head_dim = (config.n_head + 2 * config.n_local_heads) * config.head_dim
        assert total_head_dim % tp == 0
        self.wqkv = nn.Linear(config.dim, total_head_dim // tp, bias=False)
        self.wo = nn.Linear(config.dim // tp, config.dim, bias=False)
        self._init_heads(config)

    def forward(self, x: Tensor, freqs_cis: Tensor, mask: Tensor, input_pos: Optional[Tensor] = None) -> Tensor:
        bsz, seqlen, _ = x.shape
        x = x.contiguous()
        qkv = _hip.module_linear(x, self.wqkv, x.new_empty(bsz, seqlen, self.wqkv.out_features))
        y = self._attend(qkv, bsz, seqlen, freqs_cis, input_pos)
        return _hip.module_linear(y, self.wo, x.new_empty(bsz, seqlen, self.wo.out_features))


class FuseAttentionMLP(_AttentionCore):
    """Parallel block: one projection wqkv1 with rows [q; k; v; up; gate], then
    w2(silu(gate) * up) + wo(attention)."""

    def __init__(self, config):
        super().__init__()
        tp = config.tp_world_size
        total_head_dim = (config.n_head + 2 * config.n_local_heads) * config.head_dim
        assert total_head_dim % tp == 0
        assert config.intermediate_size % tp == 0
        self.wqkv1 = nn.Linear(config.dim, total_head_dim // tp + 2 * config.intermediate_size // tp, bias=False)
        self.wo = nn.Linear(config.dim // tp, config.dim, bias=False)
        self.w2 = nn.Linear(config.intermediate_size // tp, config.dim, bias=False)
        self.intermediate_size = config.intermediate_size // tp
        self._init_heads(config)

    def forward(self, x: Tensor, freqs_cis: Tensor, mask: Tensor, input_pos: Optional[Tensor] = None) -> Tensor:
        bsz, seqlen, _ = x.shape
        x = x.contiguous()
        nqkv = (self.n_head + 2 * self.n_local_heads) * self.head_dim
        fused = _hip.module_linear(x, self.wqkv1, x.new_empty(bsz, seqlen, self.wqkv1.out_features))
        y = self._attend(fused, bsz, seqlen, freqs_cis, input_pos)
        a = _hip.module_linear(y, self.wo, x.new_empty(bsz, seqlen, self.wo.out_features))
        m = _hip.module_linear_swiglu(fused[..., nqkv:], self.w2, x.new_empty(bsz, seqlen, self.w2.out_features))
        return _hip.add(m, a, m)
