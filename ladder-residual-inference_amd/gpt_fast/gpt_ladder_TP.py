"""Ladder-Residual model on the gfx950 kernels.

Public surface of the reference's gpt_fast/gpt_ladder_TP.py: `GPTLadder` (:210-288) and
`LadderTransformerBlock` (:291-361) with the same children, `ModelArgs`, `transformer_configs`,
`find_multiple`.  The ladder schedule: each module (attention, then MLP) reads the residual stream
BEFORE the output of the module just ahead of it has been added; that output -- a row-parallel
partial sum, which in the reference is in flight in an asynchronous all-reduce -- is added one
module later.  Here the partial sum simply waits in a local buffer (`Workspace.a`, `Workspace.m`)
and the deferred add is fused with the next RMSNorm (lr_add_rmsnorm)."""
import torch
import torch.nn as nn
from torch import Tensor

from . import _hip
from ._model import GPTBase, Workspace
from .config import REGISTRIES, ModelArgs, find_multiple  # noqa: F401  (re-exported like the reference)
from .utils import Attention, FeedForward, RMSNorm, all_reduce_func

transformer_configs = REGISTRIES["ladder"]


class LadderTransformerBlock(nn.Module):
    def __init__(self, config: ModelArgs) -> None:
        super().__init__()
        self.attention = Attention(config)
        self.feed_forward = FeedForward(config)
        self.ffn_norm = RMSNorm(config.dim, config.norm_eps)
        self.attention_norm = RMSNorm(config.dim, config.norm_eps)
        self.semi_compiled_model = config.semi_compiled_model  # accepted; there is nothing to compile here

    def forward(self, previous_attention_out: Tensor, previous_mlp_out: Tensor, residual: Tensor, attention_handle,
                mlp_handle, input_pos: Tensor, freqs_cis: Tensor, mask: Tensor):
        """Reference signature (gpt_ladder_TP.py:312-358).  Handles are always None: nothing is in
        flight.  Returns (attention partial sum, mlp partial sum, residual, None, None)."""
        if attention_handle is not None:
            attention_handle.wait()
        residual = residual.contiguous()
        new_residual = torch.empty_like(residual)
        normed = torch.empty_like(residual)
        eps = self.attention_norm.eps
        _hip.add_rmsnorm(residual, previous_attention_out.contiguous(), None, self.attention_norm.weight, new_residual,
                         normed, eps)
        current_attention_out = self.attention(normed, freqs_cis, mask, input_pos)
        current_attention_out, attention_handle = all_reduce_func(current_attention_out, clone=False, async_op=True)

        if mlp_handle is not None:
            mlp_handle.wait()
        residual = torch.empty_like(new_residual)
        _hip.add_rmsnorm(new_residual, previous_mlp_out.contiguous(), None, self.ffn_norm.weight, residual, normed,
                         self.ffn_norm.eps)
        current_mlp_out = self.feed_forward(normed)
        current_mlp_out, mlp_handle = all_reduce_func(current_mlp_out, clone=False, async_op=True)
        return current_attention_out, current_mlp_out, residual, attention_handle, mlp_handle

    def extra_repr(self) -> str:
        return f"semi_compiled = {self.semi_compiled_model}"


class GPTLadder(GPTBase):
    family = "ladder"

    def _make_block(self, config, layer_idx):
        return LadderTransformerBlock(config)

    def _run_layers(self, ws: Workspace, pos: Tensor):
        eps = self.config.norm_eps
        pending_a = pending_m = None  # the reference starts from zero tensors; adding zero is the identity
        for blk in self.layers:
            _hip.add_rmsnorm(ws.x, pending_a, None, blk.attention_norm.weight, ws.x, ws.xn, eps)
            self._attention(ws, blk, pos, blk.attention.wqkv.weight, ws.a)
            pending_a = ws.a
            _hip.add_rmsnorm(ws.x, pending_m, None, blk.ffn_norm.weight, ws.x, ws.xn, eps)
            self._mlp(ws, blk, ws.m)
            pending_m = ws.m
        return pending_a, pending_m
