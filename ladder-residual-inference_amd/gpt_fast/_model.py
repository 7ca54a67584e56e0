"""Model skeleton shared by GPTLadder / GPTDense / GPTDesync / GPTParallel.

Module tree and public surface follow the reference (gpt_ladder_TP.py:210-288): children
`tok_embeddings`, `layers`, `norm`, `output`; `setup_caches(max_batch_size, max_seq_length)`;
`forward(idx [B, S], input_pos [S]) -> logits [B, S, V]`; `from_name`.  forward() is a fixed
sequence of libladder_hip.so launches over preallocated buffers: no allocation after the first call
for a given (B, S), no host synchronisation, positions read from the device tensor `input_pos` --
so one decode step can be captured into a hipGraph and replayed while `input_pos` and the token
buffer are advanced on the device.  The only torch kernels are dtype / layout conversions of
arguments that arrive in another form (int64 positions, a non-contiguous token tensor)."""
from typing import Dict, Optional

import torch
import torch.nn as nn
from torch import Tensor

from . import _hip
from .config import ModelArgs, find_multiple
from .utils import KVCache, RMSNorm, _pos_i32, precompute_freqs_cis


class Workspace:
    """Activation buffers for one (batch, seq) shape, all bf16 [rows, *]."""

    def __init__(self, cfg: ModelArgs, B: int, S: int, fused_width: int, device, dtype, smax: int, all_logits: bool):
        rows = B * S
        D, hd = cfg.dim, cfg.head_dim
        e = lambda *shape: torch.empty(*shape, dtype=dtype, device=device)
        self.B, self.S, self.rows = B, S, rows
        self.x = e(rows, D)        # residual stream
        self.xn = e(rows, D)       # normed input of the current module
        self.xn2 = e(rows, D)      # the MLP's normed input, formed together with the attention's (ladder schedule)
        self.a = e(rows, D)        # attention partial sum (pending in the ladder schedule)
        self.m = e(rows, D)        # MLP partial sum
        self.qkv = e(rows, fused_width)
        self.y = e(rows, cfg.n_head_local * hd)
        self.h = e(rows, 2 * cfg.ffn_local)
        self.act = e(rows, cfg.ffn_local)   # activated MLP input where SwiGLU is not fused into the projection
        self.logits = e(B, S if all_logits else 1, cfg.output_rows)
        if S > 1 and not all_logits:
            # prefill with the head on the last position only: the B last rows are gathered out of the [B * S, D]
            # buffers with the row-gather kernel (lr_embed) into these
            self.last_rows = (torch.arange(1, B + 1, dtype=torch.int32, device=device) * S - 1).contiguous()
            self.xl, self.d1l, self.d2l, self.xnl = e(B, D), e(B, D), e(B, D), e(B, D)
        self.next_token = torch.empty(B, 1, dtype=torch.int32, device=device)
        self.next_token_valid_for = None   # set by a fused decode step that already chose the token
        self.scratch = None
        if S == 1:
            n = _hip.attn_decode_scratch_bytes(B, cfg.n_head_local, hd, smax) // 4
            self.scratch = torch.empty(n, dtype=torch.float32, device=device)


class GPTBase(nn.Module):
    family = "ladder"

    def __init__(self, config: ModelArgs) -> None:
        super().__init__()
        self.config = config
        self.tok_embeddings = nn.Embedding(config.vocab_size, config.dim)
        self.layers = nn.ModuleList(self._make_block(config, i) for i in range(config.n_layer))
        self.norm = RMSNorm(config.dim, eps=config.norm_eps)
        self.output = nn.Linear(config.dim, config.output_rows, bias=False)

        self.freqs_cis: Optional[Tensor] = None
        self.mask_cache: Optional[Tensor] = None
        self.causal_mask: Optional[Tensor] = None
        self.max_batch_size = -1
        self.max_seq_length = -1
        # False: logits for every position, as the reference returns; True: only the last position
        # of each sequence goes through the final norm and lm_head (prefill saves S-1 rows of it)
        self.last_logits_only = False
        self._ws: Dict[tuple, Workspace] = {}

    # -- construction ---------------------------------------------------------------------------
    def _make_block(self, config, layer_idx):
        raise NotImplementedError

    @classmethod
    def from_name(cls, name: str):
        from .config import args_from_name

        return cls(args_from_name(cls.family, name))

    def _fused_width(self) -> int:
        c = self.config
        return (c.n_head_local + 2 * c.n_kv_local) * c.head_dim

    # -- caches ---------------------------------------------------------------------------------
    def setup_caches(self, max_batch_size, max_seq_length):
        if self.max_seq_length >= max_seq_length and self.max_batch_size >= max_batch_size:
            return
        cfg = self.config
        if cfg.head_dim not in (64, 128):
            raise NotImplementedError(f"head_dim {cfg.head_dim}: the attention kernels are built for 64 and 128")
        if max_seq_length > cfg.block_size:
            # the RoPE table has block_size rows: the reference fails with an index error at the first position
            # beyond it (gpt_ladder_TP.py:255); here the mistake is reported before anything is allocated
            raise ValueError(f"max_seq_length {max_seq_length} exceeds the model's block_size {cfg.block_size}")
        max_seq_length = find_multiple(max_seq_length, 8)
        self.max_seq_length = max_seq_length
        self.max_batch_size = max_batch_size
        dtype = self.output.weight.dtype
        # for weight-only quantised layers the model dtype is the scales' (gpt_ladder_TP.py:232-237)
        if hasattr(self.output, "scales"):
            dtype = self.output.scales.dtype
        device = self.output.weight.device
        if dtype != torch.bfloat16:
            raise NotImplementedError(f"the HIP kernels compute in bfloat16 storage; model dtype is {dtype}")
        for b in self.layers:
            b.attention.kv_cache = KVCache(max_batch_size, max_seq_length, cfg.n_kv_local, cfg.head_dim, dtype).to(device)
        self.freqs_cis = precompute_freqs_cis(cfg.block_size, cfg.head_dim, cfg.rope_base, dtype,
                                              cfg.rope_scaling).to(device)
        # kept for API compatibility (the kernels derive visibility from input_pos)
        self.causal_mask = torch.tril(torch.ones(max_seq_length, max_seq_length, dtype=torch.bool, device=device))
        self._ws.clear()
        _hip.device_error_word(device)  # exists before any step is captured into a graph

    def check_device_errors(self):
        """Synchronises, then raises LadderHipError if a kernel of an earlier call reported a condition
        only the device can see: a position outside the KV cache / RoPE table (the reference raises
        an index error there), or an expired wait inside the one-kernel decode step.  benchmark.py
        calls it after every generation, next to the synchronisation it does anyway."""
        fused = [f for f in getattr(self, "_fused", {}).values() if f is not None]
        _hip.raise_on_device_error(self.output.weight.device, fused)

    def release_workspace(self):
        self._ws.clear()

    def _workspace(self, B: int, S: int) -> Workspace:
        key = (B, S, self.last_logits_only)
        ws = self._ws.get(key)
        if ws is None:
            w = self.output.weight
            ws = Workspace(self.config, B, S, self._fused_width(), w.device, self.norm.weight.dtype, self.max_seq_length,
                           not self.last_logits_only)
            if S > 1:  # keep at most one prefill-sized workspace alive
                for k in [k for k in self._ws if k[1] > 1]:
                    del self._ws[k]
            self._ws[key] = ws
        return ws

    # -- forward --------------------------------------------------------------------------------
    def forward(self, idx: Tensor, input_pos: Optional[Tensor] = None) -> Tensor:
        assert self.freqs_cis is not None, "Caches must be initialized first"
        B, S = idx.shape
        assert B <= self.max_batch_size and input_pos.shape[-1] == S
        pos = _pos_i32(input_pos)
        ws = self._workspace(B, S)
        ws.next_token_valid_for = None
        _hip.embed(self.tok_embeddings.weight, idx.contiguous(), ws.x)
        final_d1, final_d2 = self._run_layers(ws, pos)
        cfg = self.config
        if self.last_logits_only and S > 1:
            # only row S-1 of each sequence feeds the head: gather those B rows, then norm + lm_head
            last = lambda t, out: None if t is None else _hip.embed(t.view(B * S, -1), ws.last_rows, out)
            _hip.add_rmsnorm(last(ws.x, ws.xl), last(final_d1, ws.d1l), last(final_d2, ws.d2l), self.norm.weight, None,
                             ws.xnl, cfg.norm_eps)
            _hip.module_linear(ws.xnl, self.output, ws.logits.view(B, -1))
        else:
            _hip.add_rmsnorm(ws.x, final_d1, final_d2, self.norm.weight, None, ws.xn, cfg.norm_eps)
            _hip.module_linear(ws.xn, self.output, ws.logits.view(B * S, -1))
        return ws.logits

    def _run_layers(self, ws: Workspace, pos: Tensor):
        """Runs all blocks on ws.x; returns up to two tensors still to be added to ws.x before the
        final norm (the ladder's two stragglers), or (None, None)."""
        raise NotImplementedError

    # -- shared pieces of the block schedules -----------------------------------------------------
    # decode batches from which single projections go to the weight-streaming bands (one row: the matrix-vector kernel
    # is the faster one -- dense family on the 70B rank shard, ms per step at batch 1 / 4: 5.7 / 8.5 without bands,
    # 6.1 / 6.2 with)
    band_rows_from = 2

    def _decode_bands(self, ws: Workspace, *linears) -> bool:
        """A decode step of up to 64 rows on bf16 weights: every projection of a block is a launch of the
        weight-streaming kernel (lr_linear_multi), the q/k/v one rotating and caching on its way out and the up/gate one
        storing silu(gate) * up -- also below 5 rows, where lr_linear alone would pick the matrix-vector kernel: fewer
        launches per block weigh more than the kernel.  (`linears`: the modules
        in question; weight-only quantised ones have kernels of their own.)"""
        return ws.S == 1 and self.band_rows_from <= ws.B <= 64 and not any(hasattr(m, "scales") for m in linears)

    def _attention(self, ws: Workspace, blk, pos: Tensor, wqkv: nn.Module, out: Tensor, roped: bool = False):
        """ws.xn -> fused projection -> RoPE + cache write -> attention -> wo -> out (partial sum).
        wqkv None: ws.qkv already holds the projection (roped: rotated, with k and v already in the cache).
        out None: stop at the attention output ws.y."""
        cfg = self.config
        B, S = ws.B, ws.S
        Hq, Hkv, hd = cfg.n_head_local, cfg.n_kv_local, cfg.head_dim
        kc, vc = blk.attention.kv_cache.k_cache, blk.attention.kv_cache.v_cache
        bands = self._decode_bands(ws, blk.attention.wo, *(() if wqkv is None else (wqkv,)))
        if wqkv is not None and bands and not roped:
            _hip.linear_multi((ws.xn, wqkv.weight, ws.qkv, _hip.rope_kv_epilogue(self.freqs_cis, pos, kc, vc, Hq, Hkv, hd)))
            roped = True
        elif (wqkv is not None and S > 1 and not roped and not hasattr(wqkv, "scales")
              and wqkv.weight.shape[0] == (Hq + 2 * Hkv) * hd):   # (not the parallel family's wider projection)
            # prefill: the projection rotates q and caches rotated k and v on its way out (one launch of the GEMM)
            _hip.linear_rope_kv(ws.xn, wqkv.weight, ws.qkv, self.freqs_cis, pos, kc, vc, B, S, Hq, Hkv, hd)
            roped = True
        elif wqkv is not None:
            _hip.module_linear(ws.xn, wqkv, ws.qkv)
        if not roped:
            _hip.rope_kv_write(ws.qkv, self.freqs_cis, False, pos, kc, vc, B, S, Hq, Hkv, hd)
        if S == 1:
            _hip.attn_decode(ws.qkv, kc, vc, pos, ws.y, ws.scratch, B, Hq, Hkv, hd)
        else:
            _hip.attn_prefill(ws.qkv, kc, vc, pos, ws.y, B, S, Hq, Hkv, hd)
        if out is None:
            return
        if bands:
            _hip.linear_multi((ws.y, blk.attention.wo.weight, out, _hip.EPI_NONE))
        else:
            _hip.module_linear(ws.y, blk.attention.wo, out)

    def _mlp(self, ws: Workspace, blk, out: Tensor, xn: Optional[Tensor] = None):
        ff = blk.feed_forward
        xin = ws.xn if xn is None else xn
        if self._decode_bands(ws, ff.w1, ff.w2):
            _hip.linear_multi((xin, ff.w1.weight, ws.act, _hip.EPI_SWIGLU))
            _hip.linear_multi((ws.act, ff.w2.weight, out, _hip.EPI_NONE))
            return
        if xin.shape[0] > 4 and not hasattr(ff.w1, "scales"):
            # the activation in the first projection's epilogue; up to 4 rows it is fused into w2's GEMV instead
            _hip.linear_swiglu_out(xin, ff.w1.weight, ws.act, ws.h)
            _hip.module_linear(ws.act, ff.w2, out)
            return
        _hip.module_linear(xin, ff.w1, ws.h)
        _hip.module_linear_swiglu(ws.h, ff.w2, out, ws.act)

    # -- greedy decoding helper ---------------------------------------------------------------------
    def greedy_next(self, logits: Tensor) -> Tensor:
        """argmax of the last position of `logits` [B, S, V] -> int32 [B, 1] (lowest index on ties)."""
        B = logits.shape[0]
        ws = self._ws.get((B, 1, self.last_logits_only)) or next(iter(self._ws.values()))
        out = ws.next_token if ws.next_token.shape[0] == B else torch.empty(B, 1, dtype=torch.int32,
                                                                            device=logits.device)
        return _hip.argmax(logits[:, -1], out)

    def sample_next(self, logits: Tensor, temperature: float, top_k) -> tuple:
        """benchmark.py:58-77 on the last position of bf16 `logits` [B, S, V] -> (int32 [B, 1], probs [B, V]).
        The Exp(1) noise comes from torch's generator exactly as in the reference (same shape and dtype)."""
        last = logits[:, -1]
        probs = torch.empty(last.shape, dtype=last.dtype, device=last.device)
        noise = torch.empty_like(probs).exponential_(1)
        out = torch.empty(last.shape[0], 1, dtype=torch.int32, device=last.device)
        _hip.sample_topk(last, noise, temperature, top_k, out, probs)
        return out, probs
