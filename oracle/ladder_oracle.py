"""CPU restatement of the per-rank forward pass of the Ladder-Residual reference.

TEST INFRASTRUCTURE ONLY.  This module is the checker: it may be imported by
tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg, and by
nothing else.  The product (the gpt_fast package next to the HIP sources) never
imports it and has no CPU fallback.

It restates, in plain eager PyTorch with no third-party kernels, no
torch.distributed and no module state, the maths of

  gpt_fast/gpt_ladder_TP.py:225-284, 312-358   caches, forward, ladder block schedule
  gpt_fast/gpt_dense_TP.py:274-284             dense block
  gpt_fast/gpt_desync_TP.py:319-323, 350-384   desync block
  gpt_fast/gpt_parallel_TP.py:214-226          parallel block
  gpt_fast/utils.py:43-59                      KV cache update
  gpt_fast/utils.py:62-78                      RMSNorm (the in-repo formula at :68-74)
  gpt_fast/utils.py:81-117                     RoPE table (+ Llama-3.1 scaling)
  gpt_fast/utils.py:120-132                    interleaved-pair RoPE
  gpt_fast/utils.py:135-149                    SwiGLU feed-forward
  gpt_fast/utils.py:187-198, 247-258           attention, non-flash branch
  gpt_fast/utils.py:305-387                    fused attention+MLP of the parallel block
  gpt_fast/utils.py:390-397                    all-reduce  -> identity (partial sums stay local)
  benchmark.py:58-164                          sampling / prefill / decode loop (greedy added)
  gpt_fast/gpt_ladder_TP.py:233-237            hook for weight-only quantised linears (fp8 form restated)

Every tensor is rounded to the model dtype exactly where the eager reference
rounds it: after each add, after the normalisation and again after the gain,
after every linear, after RoPE, after silu and after the gate product, after
attention.  Sums accumulate in fp32 (fp32 inputs: plain fp32).

A "rank shard" is expressed by OracleConfig.tp_world_size: per-rank sizes are the
global ones divided by it, exactly as the reference constructs its layers
(utils.py:142-143, 165-166, 174-176), and the all-reduce is the identity.

Pinning status (tests/test_oracle_*.py): every function below is pinned against a
closed form, a library routine or brute force in fp64.  The reference holds no
golden vectors, fixtures or tests for this path, and its RMSNorm eager branch
calls the un-vendored third-party liger_kernel (version not pinned by the
reference): bit-level parity with *that* kernel is "parity unpinned"; the in-repo
formula utils.py:68-74 is what is restated here.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn.functional as F

Tensor = torch.Tensor


def find_multiple(n: int, k: int) -> int:
    """gpt_ladder_TP.py:20-23."""
    return n if n % k == 0 else n + k - (n % k)


@dataclass
class OracleConfig:
    """Hyper-parameters, global (un-sharded) sizes.  gpt_ladder_TP.py:32-57."""

    block_size: int = 2048
    vocab_size: int = 32000
    n_layer: int = 32
    n_head: int = 32
    dim: int = 4096
    intermediate_size: Optional[int] = None
    n_local_heads: int = -1
    rope_base: float = 10000
    norm_eps: float = 1e-5
    rope_scaling: Optional[dict] = None
    # desync only (gpt_desync_TP.py:44-45, 59-60)
    reduce_pattern: Optional[List[Dict[str, bool]]] = None
    force_disable_last_all_reduce: bool = False
    # layers that run the ladder schedule (None: all); the others are dense -- the partial-ladder wiring of
    # hf_modeling_utils/modeling_llama_ladder.py:889-948
    ladder_layers: Optional[List[int]] = None
    # rank shard: sizes are divided by this; no collective is issued
    tp_world_size: int = 1
    # lm_head rows kept by this rank (None: full vocab, as the reference does)
    vocab_shard: Optional[int] = None

    def __post_init__(self):
        if self.n_local_heads == -1:
            self.n_local_heads = self.n_head
        if self.intermediate_size is None:
            self.intermediate_size = find_multiple(int(2 * (4 * self.dim) / 3), 256)
        assert self.dim % self.n_head == 0
        tp = self.tp_world_size
        assert self.dim % tp == 0 and self.intermediate_size % tp == 0
        assert self.n_head % tp == 0 and self.n_local_heads % tp == 0
        if self.reduce_pattern is None:
            self.reduce_pattern = [{"attention": False, "mlp": True} for _ in range(self.n_layer)]

    # per-rank sizes
    @property
    def head_dim(self) -> int:
        return self.dim // self.n_head

    @property
    def hq(self) -> int:
        return self.n_head // self.tp_world_size

    @property
    def hkv(self) -> int:
        return self.n_local_heads // self.tp_world_size

    @property
    def ffn(self) -> int:
        return self.intermediate_size // self.tp_world_size

    @property
    def out_rows(self) -> int:
        return self.vocab_size if self.vocab_shard is None else self.vocab_shard


# --------------------------------------------------------------------------------------
# parameters
# --------------------------------------------------------------------------------------

def param_shapes(cfg: OracleConfig, family: str = "ladder") -> List[Tuple[str, Tuple[int, ...]]]:
    """State-dict names and per-rank shapes in module registration order.

    Names follow the reference modules: gpt_ladder_TP.py:215-218, 294-297,
    utils.py:142-143, 165-166 (277-283 for the parallel block's fused wqkv1)."""
    D, hd = cfg.dim, cfg.head_dim
    qkv = (cfg.hq + 2 * cfg.hkv) * hd
    out = [("tok_embeddings.weight", (cfg.vocab_size, D))]
    for i in range(cfg.n_layer):
        p = f"layers.{i}."
        if family == "parallel":
            out += [
                (p + "attention.wqkv1.weight", (qkv + 2 * cfg.ffn, D)),
                (p + "attention.wo.weight", (D, cfg.hq * hd)),
                (p + "attention.w2.weight", (D, cfg.ffn)),
                (p + "attention_norm.weight", (D,)),
            ]
        else:
            out += [
                (p + "attention.wqkv.weight", (qkv, D)),
                (p + "attention.wo.weight", (D, cfg.hq * hd)),
                (p + "feed_forward.w1.weight", (2 * cfg.ffn, D)),
                (p + "feed_forward.w2.weight", (D, cfg.ffn)),
                (p + "ffn_norm.weight", (D,)),
                (p + "attention_norm.weight", (D,)),
            ]
    out += [("norm.weight", (D,)), ("output.weight", (cfg.out_rows, D))]
    return out


def init_params(cfg: OracleConfig, family: str = "ladder", seed: int = 0, dtype=torch.float32,
                device="cpu", std: float = 0.02) -> Dict[str, Tensor]:
    """N(0, std) for EVERY parameter, norm gains included (benchmark.py:242-243).

    The reference sets no seed; the seeded generator is this build's addition so
    that two implementations can be given identical bits."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    params = {}
    for name, shape in param_shapes(cfg, family):
        t = torch.empty(shape, dtype=torch.float32 if str(device) == "cpu" else dtype, device=device)
        t.normal_(0.0, std, generator=g)
        params[name] = t.to(dtype)
    return params


# --------------------------------------------------------------------------------------
# ops
# --------------------------------------------------------------------------------------

def rms_norm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    """utils.py:68-74: normalise in fp32, round to x.dtype, THEN multiply by the gain."""
    xf = x.float()
    n = (xf * torch.rsqrt(torch.mean(xf * xf, dim=-1, keepdim=True) + eps)).type_as(x)
    return n * weight


# --- weight-only fp8 linears.  The reference only leaves the hook of gpt-fast's weight-only quantisation
# (gpt_ladder_TP.py:233-237: a quantised nn.Linear replacement keeps `weight` in the narrow type and a
# per-output-row `scales` in the model dtype); the arithmetic restated here is that scheme's,
#     y = F.linear(x, weight.to(x.dtype)) * scales,
# with e4m3 weights.  No reference file carries the quantiser or the quantised forward, so parity at
# this boundary is "parity unpinned"; the functions are pinned by closed forms (tests/test_oracle_ops.py).
FP8_MAX = 448.0  # largest finite float8_e4m3fn


def quantize_fp8_rowwise(w: Tensor, scale_dtype=torch.bfloat16) -> Tuple[Tensor, Tensor]:
    """w [N, K] -> (float8_e4m3fn [N, K], scales [N] in scale_dtype): row n is stored as w[n] / scales[n]
    with scales[n] = max|w[n]| / 448 rounded to scale_dtype (rows of zeros get scale 1)."""
    amax = w.float().abs().amax(dim=1)
    scales = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax)).to(scale_dtype)
    q = (w.float() / scales.float()[:, None]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, scales


def linear_fp8(x: Tensor, w8: Tensor, scales: Tensor) -> Tensor:
    """F.linear(x, w8.to(x.dtype)) * scales: the e4m3 -> bf16 conversion is exact, the product is rounded to
    x.dtype by the matmul and once more after the scaling."""
    return F.linear(x, w8.to(x.dtype)) * scales.to(x.dtype)


def linear(P: Dict[str, Tensor], name: str, x: Tensor) -> Tensor:
    """nn.Linear without bias on parameter `name` of P; the weight-only fp8 form if P holds
    `<module>.scales` beside `<module>.weight`."""
    scales = P.get(name[: -len("weight")] + "scales")
    if scales is not None:
        return linear_fp8(x, P[name], scales)
    return F.linear(x, P[name])


def quantize_params_fp8(P: Dict[str, Tensor]) -> Dict[str, Tensor]:
    """Every projection (wqkv, wqkv1, wo, w1, w2, output) of a parameter dict in the weight-only fp8 form;
    norm gains and the embedding table stay as they are."""
    out = {}
    for name, w in P.items():
        if w.dim() == 2 and name != "tok_embeddings.weight":
            out[name], out[name[: -len("weight")] + "scales"] = quantize_fp8_rowwise(w, w.dtype)
        else:
            out[name] = w
    return out


def rope_scaled_freqs(freqs: Tensor, rope_scaling: dict) -> Tensor:
    """Llama-3.1 wavelength-banded frequency scaling.  utils.py:81-100."""
    factor = rope_scaling["factor"]
    lo = rope_scaling["low_freq_factor"]
    hi = rope_scaling["high_freq_factor"]
    old_len = rope_scaling["original_max_position_embeddings"]
    lo_wavelen = old_len / lo
    hi_wavelen = old_len / hi
    out = []
    for f in freqs:  # element by element, as the reference does (python-float maths on 0-d tensors)
        wavelen = 2 * math.pi / f
        if wavelen < hi_wavelen:
            out.append(f)
        elif wavelen > lo_wavelen:
            out.append(f / factor)
        else:
            smooth = (old_len / wavelen - lo) / (hi - lo)
            out.append((1 - smooth) * f / factor + smooth * f)
    return torch.tensor(out, dtype=freqs.dtype)


def rope_table(seq_len: int, n_elem: int, base: float = 10000, dtype=torch.bfloat16,
               rope_scaling: Optional[dict] = None) -> Tensor:
    """[seq_len, n_elem/2, 2] = (cos, sin) of t * base^(-2j/n_elem), computed in fp32 on the
    host and THEN cast to the model dtype.  utils.py:103-117."""
    freqs = 1.0 / (base ** (torch.arange(0, n_elem, 2)[: n_elem // 2].float() / n_elem))
    if rope_scaling is not None:
        freqs = rope_scaled_freqs(freqs, rope_scaling)
    t = torch.arange(seq_len)
    ang = torch.outer(t, freqs)  # int64 x fp32 -> fp32
    return torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).to(dtype)


def apply_rope(x: Tensor, freqs_cis: Tensor) -> Tensor:
    """Interleaved pairs (x[2j], x[2j+1]) rotated in fp32, result cast back.  utils.py:120-132.

    x [B, S, H, hd]; freqs_cis [S, hd/2, 2] in the model dtype (promoted to fp32 here)."""
    xs = x.float().reshape(*x.shape[:-1], -1, 2)
    fc = freqs_cis.view(1, xs.size(1), 1, xs.size(3), 2)
    x0, x1, c, s = xs[..., 0], xs[..., 1], fc[..., 0], fc[..., 1]
    out = torch.stack([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1)
    return out.flatten(3).type_as(x)


def kv_update(k_cache: Tensor, v_cache: Tensor, input_pos: Tensor, k: Tensor, v: Tensor) -> None:
    """cache[:, :, input_pos] = value, in place.  utils.py:50-59.  caches [B, Hkv, Smax, hd]."""
    assert input_pos.shape[0] == k.shape[2]
    bsz = k.shape[0]
    k_cache[:bsz, :, input_pos] = k
    v_cache[:bsz, :, input_pos] = v


def sdpa_math(q: Tensor, k: Tensor, v: Tensor, mask: Tensor) -> Tensor:
    """softmax(q k^T / sqrt(hd) + mask) v with GQA expansion, computed in fp32 and rounded
    once at the end -- what F.scaled_dot_product_attention's math backend (forced by
    benchmark.py:107,142) does for half-precision inputs.  utils.py:252-255.

    q [B, Hq, S, hd]; k, v [B, Hkv, Smax, hd] (the whole cache); mask [S, Smax] bool."""
    B, Hq, S, hd = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv  # q head h reads kv head h // G (repeat_interleave, utils.py:252-253)
    qf = q.float().view(B, Hkv, G, S, hd)
    kf = k.float()[:, :, None]
    vf = v.float()[:, :, None]
    s = torch.matmul(qf, kf.transpose(-1, -2)) * (1.0 / math.sqrt(hd))
    s = s.masked_fill(~mask.view(1, 1, 1, S, -1), float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.matmul(p, vf).view(B, Hq, S, hd).to(q.dtype)


@dataclass
class OracleCaches:
    """What setup_caches builds.  gpt_ladder_TP.py:225-250."""

    k: List[Tensor]
    v: List[Tensor]
    freqs_cis: Tensor
    causal_mask: Tensor
    max_seq_length: int


def setup_caches(cfg: OracleConfig, max_batch_size: int, max_seq_length: int, dtype, device="cpu") -> OracleCaches:
    smax = find_multiple(max_seq_length, 8)
    shape = (max_batch_size, cfg.hkv, smax, cfg.head_dim)
    ks = [torch.zeros(shape, dtype=dtype, device=device) for _ in range(cfg.n_layer)]
    vs = [torch.zeros(shape, dtype=dtype, device=device) for _ in range(cfg.n_layer)]
    table = rope_table(cfg.block_size, cfg.head_dim, cfg.rope_base, dtype, cfg.rope_scaling).to(device)
    mask = torch.tril(torch.ones(smax, smax, dtype=torch.bool, device=device))
    return OracleCaches(ks, vs, table, mask, smax)


def _attn_core(cfg: OracleConfig, q: Tensor, k: Tensor, v: Tensor, layer: int, caches: OracleCaches,
               freqs_cis: Tensor, mask: Tensor, input_pos: Tensor) -> Tensor:
    """utils.py:193-198, 247-257: heads view, RoPE on q and k, BHSD, cache update, SDPA, BSHD."""
    B, S, _ = q.shape
    hd = cfg.head_dim
    q = apply_rope(q.reshape(B, S, cfg.hq, hd), freqs_cis).transpose(1, 2)
    k = apply_rope(k.reshape(B, S, cfg.hkv, hd), freqs_cis).transpose(1, 2)
    v = v.reshape(B, S, cfg.hkv, hd).transpose(1, 2)
    kv_update(caches.k[layer], caches.v[layer], input_pos, k, v)
    y = sdpa_math(q, caches.k[layer][:B], caches.v[layer][:B], mask)
    return y.transpose(1, 2).contiguous().view(B, S, cfg.hq * hd)


def attention(cfg: OracleConfig, P: Dict[str, Tensor], layer: int, x: Tensor, caches: OracleCaches,
              freqs_cis: Tensor, mask: Tensor, input_pos: Tensor) -> Tensor:
    """utils.py:187-260 (non-flash).  wqkv rows are [q_local; k_local; v_local]."""
    p = f"layers.{layer}.attention."
    hd = cfg.head_dim
    q, k, v = linear(P, p + "wqkv.weight", x).split([cfg.hq * hd, cfg.hkv * hd, cfg.hkv * hd], dim=-1)
    y = _attn_core(cfg, q, k, v, layer, caches, freqs_cis, mask, input_pos)
    return linear(P, p + "wo.weight", y)  # row-parallel: a partial sum


def feed_forward(cfg: OracleConfig, P: Dict[str, Tensor], layer: int, x: Tensor) -> Tensor:
    """utils.py:145-149.  w1 rows are [up; gate]: u is the FIRST half, g the second."""
    p = f"layers.{layer}.feed_forward."
    u, g = linear(P, p + "w1.weight", x).chunk(2, dim=-1)
    return linear(P, p + "w2.weight", F.silu(g) * u)  # row-parallel: a partial sum


def fused_attention_mlp(cfg: OracleConfig, P: Dict[str, Tensor], layer: int, x: Tensor, caches: OracleCaches,
                        freqs_cis: Tensor, mask: Tensor, input_pos: Tensor) -> Tensor:
    """utils.py:305-387.  wqkv1 rows are [q; k; v; u; g]; result = w2(silu(g) u) + wo(y)."""
    p = f"layers.{layer}.attention."
    hd = cfg.head_dim
    q, k, v, u, g = linear(P, p + "wqkv1.weight", x).split(
        [cfg.hq * hd, cfg.hkv * hd, cfg.hkv * hd, cfg.ffn, cfg.ffn], dim=-1)
    y = _attn_core(cfg, q, k, v, layer, caches, freqs_cis, mask, input_pos)
    y = linear(P, p + "wo.weight", y)
    return linear(P, p + "w2.weight", F.silu(g) * u) + y


# --------------------------------------------------------------------------------------
# block schedules.  all_reduce_func (utils.py:390-397) is the identity here.
# --------------------------------------------------------------------------------------

def ladder_block(cfg, P, layer, prev_attn, prev_mlp, residual, caches, freqs_cis, mask, input_pos):
    """gpt_ladder_TP.py:312-358."""
    p = f"layers.{layer}."
    residual = residual + prev_attn                                               # :326-332
    a = attention(cfg, P, layer, rms_norm(residual, P[p + "attention_norm.weight"], cfg.norm_eps),
                  caches, freqs_cis, mask, input_pos)                             # :337
    residual = residual + prev_mlp                                                # :346-349
    m = feed_forward(cfg, P, layer, rms_norm(residual, P[p + "ffn_norm.weight"], cfg.norm_eps))  # :354
    return a, m, residual


def _prologue(P, caches, idx, input_pos):
    mask = caches.causal_mask[input_pos]          # gpt_ladder_TP.py:254 (without the two unit dims)
    freqs_cis = caches.freqs_cis[input_pos]       # :255
    x = F.embedding(idx, P["tok_embeddings.weight"])  # :256
    return x, freqs_cis, mask


def _epilogue(cfg, P, x):
    return linear(P, "output.weight", rms_norm(x, P["norm.weight"], cfg.norm_eps))  # :282-283


def forward_ladder(cfg: OracleConfig, P: Dict[str, Tensor], caches: OracleCaches, idx: Tensor,
                   input_pos: Tensor) -> Tensor:
    """gpt_ladder_TP.py:252-284.  idx [B, S] -> logits [B, S, out_rows]."""
    x, freqs_cis, mask = _prologue(P, caches, idx, input_pos)
    pa = torch.zeros_like(x)
    pm = torch.zeros_like(x)
    for i in range(cfg.n_layer):
        if cfg.ladder_layers is None or i in cfg.ladder_layers:
            pa, pm, x = ladder_block(cfg, P, i, pa, pm, x, caches, freqs_cis, mask, input_pos)
        else:
            # dense layer of a partial-ladder model (modeling_llama_ladder.py:614-637, 889-948), in the
            # pending-sum form: it reads the full sum, adds its attention output at once and leaves its MLP
            # output pending (a following ladder layer's attention must not see it, :644)
            p = f"layers.{i}."
            x = x + pa + pm
            x = x + attention(cfg, P, i, rms_norm(x, P[p + "attention_norm.weight"], cfg.norm_eps),
                              caches, freqs_cis, mask, input_pos)
            pm = feed_forward(cfg, P, i, rms_norm(x, P[p + "ffn_norm.weight"], cfg.norm_eps))
            pa = torch.zeros_like(x)
    x = x + pa + pm                                                                # :280
    return _epilogue(cfg, P, x)


def forward_dense(cfg, P, caches, idx, input_pos) -> Tensor:
    """gpt_dense_TP.py:227-237, 281-282."""
    x, freqs_cis, mask = _prologue(P, caches, idx, input_pos)
    for i in range(cfg.n_layer):
        p = f"layers.{i}."
        x = x + attention(cfg, P, i, rms_norm(x, P[p + "attention_norm.weight"], cfg.norm_eps),
                          caches, freqs_cis, mask, input_pos)
        x = x + feed_forward(cfg, P, i, rms_norm(x, P[p + "ffn_norm.weight"], cfg.norm_eps))
    return _epilogue(cfg, P, x)


def desync_flags(cfg: OracleConfig, layer: int) -> Tuple[bool, bool]:
    """gpt_desync_TP.py:319-323."""
    do_attn = cfg.reduce_pattern[layer]["attention"]
    do_mlp = layer == cfg.n_layer - 1 or cfg.reduce_pattern[layer]["mlp"]
    if layer == cfg.n_layer - 1 and cfg.force_disable_last_all_reduce:
        do_mlp = False
    return do_attn, do_mlp


def forward_desync(cfg, P, caches, idx, input_pos) -> Tensor:
    """gpt_desync_TP.py:294-304, 366-382: the residual is pre-divided by tp where a reduce follows."""
    x, freqs_cis, mask = _prologue(P, caches, idx, input_pos)
    tp = cfg.tp_world_size
    for i in range(cfg.n_layer):
        p = f"layers.{i}."
        do_attn, do_mlp = desync_flags(cfg, i)
        r = x
        x = attention(cfg, P, i, rms_norm(x, P[p + "attention_norm.weight"], cfg.norm_eps),
                      caches, freqs_cis, mask, input_pos)
        x = x + r / tp if do_attn else x + r
        r = x
        x = feed_forward(cfg, P, i, rms_norm(x, P[p + "ffn_norm.weight"], cfg.norm_eps))
        x = x + r / tp if do_mlp else x + r
    return _epilogue(cfg, P, x)


def forward_parallel(cfg, P, caches, idx, input_pos) -> Tensor:
    """gpt_parallel_TP.py:178-188, 220-224: one norm, fused projection, y + x."""
    x, freqs_cis, mask = _prologue(P, caches, idx, input_pos)
    for i in range(cfg.n_layer):
        p = f"layers.{i}."
        y = fused_attention_mlp(cfg, P, i, rms_norm(x, P[p + "attention_norm.weight"], cfg.norm_eps),
                                caches, freqs_cis, mask, input_pos)
        x = y + x
    return _epilogue(cfg, P, x)


FORWARD = {"ladder": forward_ladder, "dense": forward_dense, "desync": forward_desync, "parallel": forward_parallel}


# --------------------------------------------------------------------------------------
# generation loop
# --------------------------------------------------------------------------------------

def greedy(logits: Tensor) -> Tensor:
    """argmax of the last position, first maximum on ties -> int32 [B, 1].  Stands where
    benchmark.py:73-77 samples; the parity contract of this build is greedy decoding."""
    return torch.argmax(logits[:, -1], dim=-1, keepdim=True).to(torch.int32)


def sample_topk(last_logits: Tensor, noise: Tensor, temperature: float = 1.0, top_k: Optional[int] = None):
    """benchmark.py:58-77 (sample / logits_to_probs / multinomial_sample_one_no_sync) on the logits of
    the last position [B, V], with the Exp(1) draws of :59 passed in as `noise` [B, V] so that a run can
    be repeated:  scale by 1 / max(T, 1e-5) (:64), everything below the top_k-th largest value to -inf
    (:66-69, ties with the pivot stay), softmax (:70), token = argmax(probs / noise) (:60).
    Works in the dtype of `last_logits` (the reference samples from bf16 logits), on its device.
    Returns (int32 [B, 1], probs [B, V])."""
    s = last_logits / max(temperature, 1e-5)
    if top_k is not None:
        k = min(int(top_k), s.size(-1))
        pivot = torch.topk(s, k, dim=-1).values[..., k - 1:k]
        s = s.masked_fill(s < pivot, float("-inf"))
    probs = torch.softmax(s, dim=-1)
    token = torch.argmax(probs / noise, dim=-1, keepdim=True).to(torch.int32)
    return token, probs


@torch.no_grad()
def generate(cfg: OracleConfig, P: Dict[str, Tensor], prompt: Tensor, max_new_tokens: int, batch_size: int,
             family: str = "ladder", caches: Optional[OracleCaches] = None, forced: Optional[Tensor] = None,
             timers: Optional[dict] = None):
    """benchmark.py:118-164 with greedy sampling.

    prompt [T] int64; the same prompt in every batch row (:136).  Returns
    (tokens [B, max_new_tokens] int32, logits [max_new_tokens, B, out_rows]).
    forced [B, max_new_tokens]: teacher forcing -- feed these tokens instead of the oracle's own
    choices (the returned tokens are still the oracle's argmax at each step)."""
    import time

    fwd = FORWARD[family]
    dev = prompt.device
    dtype = P["output.scales"].dtype if "output.scales" in P else P["output.weight"].dtype   # gpt_ladder_TP.py:232-237
    T = prompt.numel()
    if caches is None:
        caches = setup_caches(cfg, batch_size, min(T + max_new_tokens, cfg.block_size), dtype, dev)
    x = prompt.view(1, -1).repeat(batch_size, 1)
    t0 = time.perf_counter()
    logits = fwd(cfg, P, caches, x, torch.arange(0, T, device=dev))
    if dev.type == "cuda":
        torch.cuda.synchronize()
    t1 = time.perf_counter()
    toks = [greedy(logits)]
    all_logits = [logits[:, -1].clone()]
    input_pos = torch.tensor([T], device=dev, dtype=torch.int)
    for i in range(max_new_tokens - 1):                                            # :156 -> :105-113
        cur = toks[-1] if forced is None else forced[:, i:i + 1].to(torch.int32)
        logits = fwd(cfg, P, caches, cur, input_pos)
        toks.append(greedy(logits))
        all_logits.append(logits[:, -1].clone())
        input_pos = input_pos + 1
    if dev.type == "cuda":
        torch.cuda.synchronize()
    t2 = time.perf_counter()
    if timers is not None:
        timers["prefill_latency"] = t1 - t0
        timers["decode_latency"] = t2 - t1
    return torch.cat(toks, dim=1), torch.stack(all_logits, dim=0)
