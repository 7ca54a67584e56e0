"""PaLM-style parallel attention + MLP block on the gfx950 kernels.

Public surface of the reference's gpt_fast/gpt_parallel_TP.py (`GPTParallel` :136-192,
`ParallelTransformerBlock` :195-229): one RMSNorm and one fused projection `wqkv1` per layer,
y = w2(silu(g) * u) + wo(attention), x = y + x.  As in the dense family, a semi-compiled shard
that is not rank 0 carries no residual (:205-206)."""
import torch
import torch.nn as nn
from torch import Tensor

from . import _hip
from ._model import GPTBase, Workspace
from .config import REGISTRIES, ModelArgs, find_multiple  # noqa: F401
from .utils import FuseAttentionMLP, RMSNorm, all_reduce_func

transformer_configs = REGISTRIES["parallel"]


class ParallelTransformerBlock(nn.Module):
    def __init__(self, config: ModelArgs) -> None:
        super().__init__()
        self.attention = FuseAttentionMLP(config)
        self.attention_norm = RMSNorm(config.dim, config.norm_eps)
        self.semi_compiled_model = config.semi_compiled_model
        self.keeps_residual = not (config.semi_compiled_model and config.tp_rank != 0)

    def forward(self, x: Tensor, input_pos: Tensor, freqs_cis: Tensor, mask: Tensor) -> Tensor:
        x = x.contiguous()
        y = self.attention(self.attention_norm(x), freqs_cis, mask, input_pos)
        y = all_reduce_func(y, clone=False)[0]
        return _hip.add(y, x, torch.empty_like(y)) if self.keeps_residual else y

    def extra_repr(self) -> str:
        return f"semi_compiled = {self.semi_compiled_model}"


class GPTParallel(GPTBase):
    family = "parallel"
    band_rows_from = 1   # six launches per block instead of nine also pay for a single row (5.6 -> 5.0 ms, 70B shard)

    def _make_block(self, config, layer_idx):
        return ParallelTransformerBlock(config)

    def _fused_width(self) -> int:
        return super()._fused_width() + 2 * self.config.ffn_local

    def _run_layers(self, ws: Workspace, pos: Tensor):
        cfg = self.config
        nqkv = (cfg.n_head_local + 2 * cfg.n_kv_local) * cfg.head_dim
        att0 = self.layers[0].attention
        if self._decode_bands(ws, att0.wqkv1, att0.wo, att0.w2):
            return self._run_layers_decode(ws, pos, nqkv)
        for blk in self.layers:
            att = blk.attention
            _hip.add_rmsnorm(ws.x, None, None, blk.attention_norm.weight, None, ws.xn, cfg.norm_eps)
            self._attention(ws, blk, pos, att.wqkv1, ws.a)   # ws.qkv holds [q | k | v | u | g]
            _hip.module_linear_swiglu(ws.qkv[:, nqkv:], att.w2, ws.m, ws.act)
            _hip.add(ws.m, ws.a, ws.m)                               # w2(...) + wo(...)
            if blk.keeps_residual:
                _hip.add(ws.m, ws.x, ws.x)                           # y + x
            else:
                ws.x.copy_(ws.m)
        return None, None

    def _run_layers_decode(self, ws: Workspace, pos: Tensor, nqkv: int):
        """Decode step through the weight-streaming bands.  The rows of the fused input weight are two projections
        of the same input: [q | k | v], rotated and cached on the way out, and [up | gate], stored as silu(gate) * up
        -- the second independent of the attention, so up to 16 sequences its bands share the attention's launch
        (lr_attn_decode_beside) and above that the q/k/v launch; wo and w2 share a launch; y + x is left to the next
        block's norm launch (x + y: the same sum).  Six launches per block instead of nine."""
        cfg = self.config
        Hq, Hkv, hd = cfg.n_head_local, cfg.n_kv_local, cfg.head_dim
        q = ws.qkv[:, :nqkv]
        pending = None
        for blk in self.layers:
            att, kv = blk.attention, blk.attention.kv_cache
            _hip.add_rmsnorm(ws.x, pending, None, blk.attention_norm.weight, None if pending is None else ws.x, ws.xn,
                             cfg.norm_eps)
            w = att.wqkv1.weight
            qkv = (ws.xn, w[:nqkv], q, _hip.rope_kv_epilogue(self.freqs_cis, pos, kv.k_cache, kv.v_cache, Hq, Hkv, hd))
            up_gate = (ws.xn, w[nqkv:], ws.act, _hip.EPI_SWIGLU)
            if ws.B <= 16:
                _hip.linear_multi(qkv)
                if not _hip.attn_decode_beside(q, kv.k_cache, kv.v_cache, pos, ws.y, ws.scratch, ws.B, Hq, Hkv, hd, up_gate):
                    _hip.linear_multi(up_gate)
                    _hip.attn_decode(q, kv.k_cache, kv.v_cache, pos, ws.y, ws.scratch, ws.B, Hq, Hkv, hd)
            else:
                _hip.linear_multi(qkv, up_gate)
                _hip.attn_decode(q, kv.k_cache, kv.v_cache, pos, ws.y, ws.scratch, ws.B, Hq, Hkv, hd)
            _hip.linear_multi((ws.y, att.wo.weight, ws.a, _hip.EPI_NONE), (ws.act, att.w2.weight, ws.m, _hip.EPI_NONE))
            _hip.add(ws.m, ws.a, ws.m)                               # w2(...) + wo(...)
            if blk.keeps_residual:
                pending = ws.m                                       # y + x: with the next norm
            else:
                ws.x.copy_(ws.m)
                pending = None
        return pending, None
