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
    # decode steps of batch <= 2 run as ONE persistent kernel (lr_ladder_decode_step) when the shape
    # is supported; set to False to force the per-op kernels
    use_fused_step = True

    def _make_block(self, config, layer_idx):
        return LadderTransformerBlock(config)

    def setup_caches(self, max_batch_size, max_seq_length):
        before = self.max_seq_length, self.max_batch_size
        super().setup_caches(max_batch_size, max_seq_length)
        if (self.max_seq_length, self.max_batch_size) != before:
            self._fused = {}

    def _fused_step(self, B: int):
        st = getattr(self, "_fused", None)
        if st is None:
            st = self._fused = {}
        if B not in st:
            # the one-kernel step implements the all-ladder schedule only, on bf16 weights or with every projection
            # (lm_head included) in weight-only e4m3
            kinds = {p.dtype for blk in self.layers for p in blk.state_dict().values() if p.dim() == 2}
            kinds.add(self.output.weight.dtype)
            ok = B <= 2 and self.config.ladder_layers is None and \
                kinds in ({torch.bfloat16}, {torch.float8_e4m3fn})
            st[B] = _hip.FusedLadderStep(self, B) if ok else None
            if st[B] is not None and not st[B].supported:
                st[B] = None
        return st[B]

    def forward(self, idx: Tensor, input_pos=None) -> Tensor:
        B, S = idx.shape
        if S == 1 and self.use_fused_step and B <= 2 and self.freqs_cis is not None:
            fused = self._fused_step(B)
            if fused is not None:
                return self.decode_step_fused(idx, input_pos)
        return super().forward(idx, input_pos)

    def decode_step_fused(self, idx: Tensor, input_pos: Tensor, advance: bool = False, history=None, pos0: int = 0):
        """One decode step through lr_ladder_decode_step.  Returns logits [B, 1, V]; the greedy token
        is left in the workspace's next_token buffer (see greedy_next).  With advance=True the step
        also writes the token into `idx` (must be int32), `history[:, pos - pos0]`, and bumps
        `input_pos` (must be int32) on the device."""
        B = idx.shape[0]
        fused = self._fused_step(B)
        ws = self._workspace(B, 1)
        tokens = idx if idx.dtype == torch.int32 else idx.to(torch.int32)
        pos = input_pos if input_pos.dtype == torch.int32 else input_pos.to(torch.int32)
        assert not advance or (tokens is idx and pos is input_pos), "advance needs int32 token and position buffers"
        fused.step(tokens.contiguous(), pos, ws.logits.view(B, -1), ws.next_token, advance,
                   tokens if advance else None, history, pos0)
        ws.next_token_valid_for = ws.logits
        return ws.logits

    def greedy_next(self, logits: Tensor) -> Tensor:
        ws = self._ws.get((logits.shape[0], 1, self.last_logits_only))
        if ws is not None and getattr(ws, "next_token_valid_for", None) is logits:
            return ws.next_token  # already chosen inside the fused step
        return super().greedy_next(logits)

    # Decode through the per-op kernels: run the attention chain and the MLP chain of a block on two streams.
    # Off by default: as parallel branches of a captured graph the chains do overlap, but every hand-over between
    # the two hardware queues costs more than the attention chain's latency that it hides (measured on the 70B rank
    # shard, ms per step with / without: batch 8 8.6 / 8.3, batch 64 18.2 / 18.8).  Putting one step of each chain
    # into the same grid instead (wqkv beside w1, attention beside w2) was slower still: 10.3 ms at batch 8.
    overlap_modules = False
    two_chains_from = 33   # decode batches from which the MLP chain is a parallel branch (see _run_layers_decode)

    def _run_layers_decode(self, ws: Workspace, pos: Tensor):
        """Decode step (S == 1) of an all-ladder model through the per-op kernels: one launch does both residual
        updates and both norms of a block (lr_ladder_norms: the MLP's input does not contain the block's own
        attention output), then the attention chain (wqkv, RoPE + cache write, attention, wo) and the MLP chain
        (w1, SwiGLU, w2) -- one after the other, or on two streams where the reference overlaps an all-reduce with
        the next module (gpt_ladder_TP.py:339-349)."""
        cfg = self.config
        eps = cfg.norm_eps
        main = side = None
        if self.overlap_modules:
            main = torch.cuda.current_stream()
            side = getattr(self, "_side_stream", None)
            if side is None or side.device != main.device:
                side = self._side_stream = torch.cuda.Stream(device=main.device)
        pending_a = pending_m = None
        # decode batches of up to 64 rows on bf16 weights: the block's two input projections share one launch of
        # the weight-streaming kernel (q/k/v -- rotated and cached on the way out -- next to up/gate, which stores
        # silu(gate) * up directly), and so do its two output projections (wo next to w2).  Also below 5 rows,
        # where single projections go to the matrix-vector kernel: five or six launches per block instead of nine
        # weigh more than the kernel (70B rank shard, ms per step: batch 1 4.9 / 5.5, batch 4 5.0 / 8.3)
        fp8 = hasattr(self.layers[0].attention.wqkv, "scales")
        multi = side is None and ws.B <= 64 and not fp8
        beside = multi and ws.B <= 16
        # Above 32 rows a band workgroup fills the register file of its waves but not the CU: the MLP chain (up/gate,
        # w2) runs as a second branch of the captured graph beside the attention chain (q/k/v, attention, wo) --
        # 70B rank shard, batch 64: 10.4 -> 9.9 ms per step; at batch 32 nothing moves (7.35 / 7.31), below that
        # the attention shares the up/gate launch instead
        two_chains = multi and not beside and ws.B >= self.two_chains_from
        if two_chains:
            cur = torch.cuda.current_stream()
            chain = getattr(self, "_chain_stream", None)
            if chain is None or chain.device != cur.device:
                chain = self._chain_stream = torch.cuda.Stream(device=cur.device)
        # weight-only e4m3 projections, up to 16 rows: the same two launches per block (lr_linear_fp8_multi)
        multi8 = side is None and fp8 and ws.B <= 16
        beside8 = multi8   # (declined by the library for a single row, where the projections are no bands)
        for blk in self.layers:
            _hip.ladder_norms(ws.x, pending_a, pending_m, blk.attention_norm.weight, blk.ffn_norm.weight, ws.x, ws.xn,
                              ws.xn2, eps)
            if multi:
                kv = blk.attention.kv_cache
                rope = _hip.rope_kv_epilogue(self.freqs_cis, pos, kv.k_cache, kv.v_cache, cfg.n_head_local,
                                             cfg.n_kv_local, cfg.head_dim)
                up_gate = (ws.xn2, blk.feed_forward.w1.weight, ws.act, _hip.EPI_SWIGLU)
                if beside:
                    # up to 16 rows the up/gate bands leave room for a second workgroup per CU: the attention's
                    # items run in the same launch and wait for the KV cache behind the weight stream
                    _hip.linear_multi((ws.xn, blk.attention.wqkv.weight, ws.qkv, rope))
                    beside = _hip.attn_decode_beside(ws.qkv, kv.k_cache, kv.v_cache, pos, ws.y, ws.scratch, ws.B,
                                                     cfg.n_head_local, cfg.n_kv_local, cfg.head_dim, up_gate)
                    if not beside:
                        _hip.linear_multi(up_gate)
                        self._attention(ws, blk, pos, None, None, roped=True)
                elif two_chains:
                    chain.wait_stream(cur)
                    with torch.cuda.stream(chain):
                        _hip.linear_multi(up_gate)
                        _hip.linear_multi((ws.act, blk.feed_forward.w2.weight, ws.m, _hip.EPI_NONE))
                    _hip.linear_multi((ws.xn, blk.attention.wqkv.weight, ws.qkv, rope))
                    self._attention(ws, blk, pos, None, None, roped=True)
                    _hip.linear_multi((ws.y, blk.attention.wo.weight, ws.a, _hip.EPI_NONE))
                    cur.wait_stream(chain)
                    pending_a, pending_m = ws.a, ws.m
                    continue
                else:
                    _hip.linear_multi((ws.xn, blk.attention.wqkv.weight, ws.qkv, rope), up_gate)
                    self._attention(ws, blk, pos, None, None, roped=True)
                _hip.linear_multi((ws.y, blk.attention.wo.weight, ws.a, _hip.EPI_NONE),
                                  (ws.act, blk.feed_forward.w2.weight, ws.m, _hip.EPI_NONE))
            elif multi8:
                att, ff, kv = blk.attention, blk.feed_forward, blk.attention.kv_cache
                rope = _hip.rope_kv_epilogue(self.freqs_cis, pos, kv.k_cache, kv.v_cache, cfg.n_head_local,
                                             cfg.n_kv_local, cfg.head_dim)
                qkv8 = (ws.xn, att.wqkv.weight, att.wqkv.scales, ws.qkv, rope)
                up_gate8 = (ws.xn2, ff.w1.weight, ff.w1.scales, ws.act, _hip.EPI_SWIGLU)
                if beside8:
                    _hip.linear_fp8_multi(qkv8)
                    beside8 = _hip.attn_decode_beside_fp8(ws.qkv, kv.k_cache, kv.v_cache, pos, ws.y, ws.scratch, ws.B,
                                                          cfg.n_head_local, cfg.n_kv_local, cfg.head_dim, up_gate8)
                    if not beside8:
                        _hip.linear_fp8_multi(up_gate8)
                        self._attention(ws, blk, pos, None, None, roped=True)
                else:
                    _hip.linear_fp8_multi(qkv8, up_gate8)
                    self._attention(ws, blk, pos, None, None, roped=True)
                _hip.linear_fp8_multi((ws.y, att.wo.weight, att.wo.scales, ws.a, _hip.EPI_NONE),
                                      (ws.act, ff.w2.weight, ff.w2.scales, ws.m, _hip.EPI_NONE))
            elif side is not None:
                side.wait_stream(main)
                with torch.cuda.stream(side):
                    self._mlp(ws, blk, ws.m, ws.xn2)
                self._attention(ws, blk, pos, blk.attention.wqkv, ws.a)
                main.wait_stream(side)
            else:
                self._attention(ws, blk, pos, blk.attention.wqkv, ws.a)
                self._mlp(ws, blk, ws.m, ws.xn2)
            pending_a, pending_m = ws.a, ws.m
        return pending_a, pending_m

    def _run_layers(self, ws: Workspace, pos: Tensor):
        cfg = self.config
        eps = cfg.norm_eps
        if ws.S == 1 and cfg.ladder_layers is None:
            return self._run_layers_decode(ws, pos)
        pending_a = pending_m = None  # the reference starts from zero tensors; adding zero is the identity
        if cfg.ladder_layers is None:
            # all-ladder prefill: both residual updates and both norms of a block in one pass over the rows
            # (lr_ladder_norms, as in decode: six tensor passes instead of the eight of two lr_add_rmsnorm)
            for blk in self.layers:
                _hip.ladder_norms(ws.x, pending_a, pending_m, blk.attention_norm.weight, blk.ffn_norm.weight, ws.x,
                                  ws.xn, ws.xn2, eps)
                self._attention(ws, blk, pos, blk.attention.wqkv, ws.a)
                self._mlp(ws, blk, ws.m, ws.xn2)
                pending_a, pending_m = ws.a, ws.m
            return pending_a, pending_m
        for i, blk in enumerate(self.layers):
            if cfg.is_ladder_layer(i):
                _hip.add_rmsnorm(ws.x, pending_a, None, blk.attention_norm.weight, ws.x, ws.xn, eps)
                self._attention(ws, blk, pos, blk.attention.wqkv, ws.a)
                pending_a = ws.a
                _hip.add_rmsnorm(ws.x, pending_m, None, blk.ffn_norm.weight, ws.x, ws.xn, eps)
                self._mlp(ws, blk, ws.m)
                pending_m = ws.m
            else:
                # a dense layer of a partial-ladder model (modeling_llama_ladder.py:614-637): it sees everything
                # produced so far, adds its attention output at once, and leaves its MLP output pending -- the
                # next layer adds it first (dense) or after its attention (ladder: "prev_attn_output" is this
                # layer's state before the MLP output, :644-658)
                _hip.add_rmsnorm(ws.x, pending_a, pending_m, blk.attention_norm.weight, ws.x, ws.xn, eps)
                self._attention(ws, blk, pos, blk.attention.wqkv, ws.a)
                _hip.add_rmsnorm(ws.x, ws.a, None, blk.ffn_norm.weight, ws.x, ws.xn, eps)
                self._mlp(ws, blk, ws.m)
                pending_a, pending_m = None, ws.m
        return pending_a, pending_m
