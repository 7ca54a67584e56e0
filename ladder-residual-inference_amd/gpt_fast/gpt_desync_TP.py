"""Pre-norm transformer with a per-layer all-reduce pattern, on the gfx950 kernels.

Public surface of the reference's gpt_fast/gpt_desync_TP.py (`GPTDesync` :252-308,
`DesyncTransformerBlock` :311-387).  `reduce_pattern[i]` says whether the attention / MLP output of
layer i would be all-reduced; where it would, the residual enters the add divided by the
tensor-parallel world size (:369-371, :378-380) so that the sum over ranks counts it once.  The
reduce itself is the identity here.  The "-upper-bound" configs never reduce: that is the dense
schedule with no communication at all."""
import torch
import torch.nn as nn
from torch import Tensor

from . import _hip
from ._model import GPTBase, Workspace
from .config import REGISTRIES, ModelArgs, find_multiple  # noqa: F401
from .utils import Attention, FeedForward, RMSNorm, all_reduce_func

transformer_configs = REGISTRIES["desync"]


class DesyncTransformerBlock(nn.Module):
    def __init__(self, config: ModelArgs, layer_idx: int) -> None:
        super().__init__()
        self.attention = Attention(config)
        self.feed_forward = FeedForward(config)
        self.ffn_norm = RMSNorm(config.dim, config.norm_eps)
        self.attention_norm = RMSNorm(config.dim, config.norm_eps)
        last = layer_idx == config.n_layer - 1
        self.do_attention_all_reduce = config.reduce_pattern[layer_idx]["attention"]
        self.do_mlp_all_reduce = last or config.reduce_pattern[layer_idx]["mlp"]
        if last and config.force_disable_last_all_reduce:
            self.do_mlp_all_reduce = False
        self.tp_world_size = config.tp_world_size
        self.semi_compiled_model = config.semi_compiled_model

    def forward(self, x: Tensor, input_pos: Tensor, freqs_cis: Tensor, mask: Tensor) -> Tensor:
        residual = x.contiguous()
        y = self.attention(self.attention_norm(residual), freqs_cis, mask, input_pos)
        x = _hip.add(y, residual, torch.empty_like(y), self.tp_world_size if self.do_attention_all_reduce else 1.0)
        if self.do_attention_all_reduce:
            x = all_reduce_func(x, clone=False)[0]
        residual = x
        y = self.feed_forward(self.ffn_norm(x))
        x = _hip.add(y, residual, torch.empty_like(y), self.tp_world_size if self.do_mlp_all_reduce else 1.0)
        if self.do_mlp_all_reduce:
            x = all_reduce_func(x, clone=False)[0]
        return x

    def extra_repr(self) -> str:
        return f"semi_compiled = {self.semi_compiled_model}"


class GPTDesync(GPTBase):
    family = "desync"

    def _make_block(self, config, layer_idx):
        return DesyncTransformerBlock(config, layer_idx)

    def _run_layers(self, ws: Workspace, pos: Tensor):
        eps = self.config.norm_eps
        tp = float(self.config.tp_world_size)
        pending = None   # a module output whose residual is not divided: its add rides in the next norm launch
        for blk in self.layers:
            _hip.add_rmsnorm(ws.x, pending, None, blk.attention_norm.weight, None if pending is None else ws.x, ws.xn,
                             eps)
            self._attention(ws, blk, pos, blk.attention.wqkv, ws.a)
            pending = ws.a
            if blk.do_attention_all_reduce and tp != 1.0:
                _hip.add(ws.a, ws.x, ws.x, tp)
                pending = None
            _hip.add_rmsnorm(ws.x, pending, None, blk.ffn_norm.weight, None if pending is None else ws.x, ws.xn, eps)
            self._mlp(ws, blk, ws.m)
            pending = ws.m
            if blk.do_mlp_all_reduce and tp != 1.0:
                _hip.add(ws.m, ws.x, ws.x, tp)
                pending = None
        return pending, None
