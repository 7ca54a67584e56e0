"""Test infrastructure: a plain restatement of the Hugging Face Llama-Ladder forward pass, in the HF
checkpoint's own parameter names and RoPE layout.  It exists to pin gpt_fast/checkpoint.py (name map,
q/k row re-ordering, [up; gate] order) and the partial-ladder wiring of the oracle and the HIP model.

Follows hf_modeling_utils/modeling_llama_ladder.py:
  :69-74    LlamaRMSNorm          weight * (x * rsqrt(mean(x^2) + eps))
  :195-226  rotate_half RoPE      q * cos + rotate_half(q) * sin, cos/sin = cat(freqs, freqs)
  :240-242  LlamaMLP              down(silu(gate(x)) * up(x))
  :530-577  attention             causal softmax(q k^T / sqrt(hd)) v with repeat_kv, o_proj
  :614-637  dense decoder layer   h = h + attn(norm1(h)); h = h + mlp(norm2(h))
  :641-660  ladder decoder layer  attn_out = h + attn(norm1(prev_attn_out)); mlp_out = attn_out + mlp(norm2(h))
  :889-948  layer loop            prev_attn_out starts as the embeddings; ladder_layers pick the form
No KV cache: the whole sequence is processed at once (prefill), which is all the pinning needs."""
import math

import torch
import torch.nn.functional as F


def _norm(x, w, eps):
    xf = x.float() if x.dtype != torch.float64 else x
    return w * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype)


def _rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def _attention(sd, pre, x, cos, sin, n_head, n_kv, hd):
    B, S, _ = x.shape
    q = F.linear(x, sd[pre + "q_proj.weight"]).view(B, S, n_head, hd).transpose(1, 2)
    k = F.linear(x, sd[pre + "k_proj.weight"]).view(B, S, n_kv, hd).transpose(1, 2)
    v = F.linear(x, sd[pre + "v_proj.weight"]).view(B, S, n_kv, hd).transpose(1, 2)
    q = q * cos + _rotate_half(q) * sin
    k = k * cos + _rotate_half(k) * sin
    k = k.repeat_interleave(n_head // n_kv, dim=1)
    v = v.repeat_interleave(n_head // n_kv, dim=1)
    s = q @ k.transpose(-1, -2) / math.sqrt(hd)
    s = s.masked_fill(~torch.tril(torch.ones(S, S, dtype=torch.bool)), float("-inf"))
    y = (torch.softmax(s, dim=-1) @ v).transpose(1, 2).reshape(B, S, n_head * hd)
    return F.linear(y, sd[pre + "o_proj.weight"])


def _mlp(sd, pre, x):
    return F.linear(F.silu(F.linear(x, sd[pre + "gate_proj.weight"])) * F.linear(x, sd[pre + "up_proj.weight"]),
                    sd[pre + "down_proj.weight"])


def hf_ladder_forward(sd, idx, n_layer, n_head, n_kv, rope_theta, eps, ladder_layers, inv_freq=None):
    """sd: HF-named state dict; idx [B, S] -> logits [B, S, vocab]."""
    h = F.embedding(idx, sd["model.embed_tokens.weight"])
    hd = h.shape[-1] // n_head
    S = idx.shape[1]
    if inv_freq is None:
        inv_freq = 1.0 / (rope_theta ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd))
    freqs = torch.outer(torch.arange(S, dtype=torch.float64), inv_freq.double())
    emb = torch.cat((freqs, freqs), dim=-1)
    cos, sin = emb.cos().to(h.dtype), emb.sin().to(h.dtype)
    prev_attn_out = h
    for i in range(n_layer):
        pre = f"model.layers.{i}."
        n1, n2 = sd[pre + "input_layernorm.weight"], sd[pre + "post_attention_layernorm.weight"]
        if i not in ladder_layers:
            h = h + _attention(sd, pre + "self_attn.", _norm(h, n1, eps), cos, sin, n_head, n_kv, hd)
            attn_out = h
            h = h + _mlp(sd, pre + "mlp.", _norm(h, n2, eps))
        else:
            attn_out = h + _attention(sd, pre + "self_attn.", _norm(prev_attn_out, n1, eps), cos, sin, n_head, n_kv, hd)
            h = attn_out + _mlp(sd, pre + "mlp.", _norm(h, n2, eps))
        prev_attn_out = attn_out
    return F.linear(_norm(h, sd["model.norm.weight"], eps), sd["lm_head.weight"])


def random_hf_state_dict(n_layer, n_head, n_kv, dim, ffn, vocab, seed=0, dtype=torch.float64, scale=None):
    g = torch.Generator().manual_seed(seed)
    hd = dim // n_head
    r = lambda *s: (torch.randn(*s, generator=g, dtype=torch.float64) * (scale or s[-1] ** -0.5)).to(dtype)
    sd = {"model.embed_tokens.weight": (torch.randn(vocab, dim, generator=g, dtype=torch.float64)).to(dtype),
          "model.norm.weight": (1 + 0.1 * torch.randn(dim, generator=g, dtype=torch.float64)).to(dtype),
          "lm_head.weight": r(vocab, dim)}
    for i in range(n_layer):
        p = f"model.layers.{i}."
        sd[p + "self_attn.q_proj.weight"] = r(n_head * hd, dim)
        sd[p + "self_attn.k_proj.weight"] = r(n_kv * hd, dim)
        sd[p + "self_attn.v_proj.weight"] = r(n_kv * hd, dim)
        sd[p + "self_attn.o_proj.weight"] = r(dim, n_head * hd)
        sd[p + "mlp.gate_proj.weight"] = r(ffn, dim)
        sd[p + "mlp.up_proj.weight"] = r(ffn, dim)
        sd[p + "mlp.down_proj.weight"] = r(dim, ffn)
        sd[p + "input_layernorm.weight"] = (1 + 0.1 * torch.randn(dim, generator=g, dtype=torch.float64)).to(dtype)
        sd[p + "post_attention_layernorm.weight"] = (1 + 0.1 * torch.randn(dim, generator=g, dtype=torch.float64)).to(dtype)
    return sd
