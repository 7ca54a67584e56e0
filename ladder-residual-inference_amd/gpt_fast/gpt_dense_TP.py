"""Standard pre-norm transformer on the gfx950 kernels: x += attn(norm x); x += mlp(norm x).

Public surface of the reference's gpt_fast/gpt_dense_TP.py (`GPTDense` :185-241,
`DenseTransformerBlock` :244-287).  Each residual add is fused with the RMSNorm that follows it.
With `semi_compiled_model` the reference adds the residual on tensor-parallel rank 0 only
(:256-257, :265-266) so that the sum over ranks counts it once; a shard built as rank != 0
therefore carries no residual."""
import torch
import torch.nn as nn
from torch import Tensor

from . import _hip
from ._model import GPTBase, Workspace
from .config import REGISTRIES, ModelArgs, find_multiple  # noqa: F401
from .utils import Attention, FeedForward, RMSNorm, all_reduce_func

transformer_configs = REGISTRIES["dense"]


class DenseTransformerBlock(nn.Module):
    def __init__(self, config: ModelArgs) -> None:
        super().__init__()
        self.attention = Attention(config)
        self.feed_forward = FeedForward(config)
        self.ffn_norm = RMSNorm(config.dim, config.norm_eps)
        self.attention_norm = RMSNorm(config.dim, config.norm_eps)
        self.semi_compiled_model = config.semi_compiled_model
        self.keeps_residual = not (config.semi_compiled_model and config.tp_rank != 0)

    def forward(self, x: Tensor, input_pos: Tensor, freqs_cis: Tensor, mask: Tensor) -> Tensor:
        x = x.contiguous()
        a = all_reduce_func(self.attention(self.attention_norm(x), freqs_cis, mask, input_pos), clone=False)[0]
        x = _hip.add(x, a, torch.empty_like(x)) if self.keeps_residual else a
        m = all_reduce_func(self.feed_forward(self.ffn_norm(x)), clone=False)[0]
        return _hip.add(x, m, torch.empty_like(x)) if self.keeps_residual else m

    def extra_repr(self) -> str:
        return f"semi_compiled = {self.semi_compiled_model}"


class GPTDense(GPTBase):
    family = "dense"

    def _make_block(self, config, layer_idx):
        return DenseTransformerBlock(config)

    def _run_layers(self, ws: Workspace, pos: Tensor):
        eps = self.config.norm_eps
        pending = None  # module output not yet added to the stream
        for blk in self.layers:
            if blk.keeps_residual:
                _hip.add_rmsnorm(ws.x, pending, None, blk.attention_norm.weight, ws.x, ws.xn, eps)
                self._attention(ws, blk, pos, blk.attention.wqkv, ws.a)
                _hip.add_rmsnorm(ws.x, ws.a, None, blk.ffn_norm.weight, ws.x, ws.xn, eps)
                self._mlp(ws, blk, ws.m)
                pending = ws.m
            else:  # the stream is replaced by the module output
                src = ws.x if pending is None else pending
                _hip.add_rmsnorm(src, None, None, blk.attention_norm.weight, None, ws.xn, eps)
                self._attention(ws, blk, pos, blk.attention.wqkv, ws.a)
                _hip.add_rmsnorm(ws.a, None, None, blk.ffn_norm.weight, None, ws.xn, eps)
                self._mlp(ws, blk, ws.m)
                pending = ws.m
        if pending is not None and not self.layers[-1].keeps_residual:
            ws.x.copy_(pending)
            pending = None
        return pending, None
