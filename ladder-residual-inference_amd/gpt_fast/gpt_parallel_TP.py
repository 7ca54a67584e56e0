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

    def _make_block(self, config, layer_idx):
        return ParallelTransformerBlock(config)

    def _fused_width(self) -> int:
        return super()._fused_width() + 2 * self.config.ffn_local

    def _run_layers(self, ws: Workspace, pos: Tensor):
        cfg = self.config
        nqkv = (cfg.n_head_local + 2 * cfg.n_kv_local) * cfg.head_dim
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
