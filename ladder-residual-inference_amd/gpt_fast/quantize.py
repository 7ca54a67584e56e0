"""Weight-only fp8 (e4m3) linears for decode.

The reference keeps the hook of gpt-fast's weight-only quantisation: a quantised replacement of
nn.Linear stores `weight` in the narrow type and per-output-row `scales` in the model dtype, and
setup_caches reads the model dtype from `output.scales` (gpt_ladder_TP.py:232-237).  This module
provides that replacement for float8_e4m3fn and the quantiser; the forward is
    y = F.linear(x, weight.to(x.dtype)) * scales
computed by lr_linear_fp8 (the fp8 bytes are streamed once: half the HBM traffic of bf16 decode).
A ladder model whose projections are all quantised (lm_head included) decodes at batch 1 and 2 through the
one-kernel step on e4m3 weights (lr_ladder_decode_step_fp8; _hip.pack_fp8_linear lays a module's bytes and
scales out the way it reads them); other batch sizes, other families and models with a bf16 lm_head go
through the per-op fp8 kernels (lr_linear_fp8, lr_linear_fp8_multi, lr_attn_decode_beside_fp8)."""
import torch
import torch.nn as nn

from . import _hip

FP8_MAX = 448.0  # largest finite float8_e4m3fn


def quantize_fp8_rowwise(w: torch.Tensor, scale_dtype=torch.bfloat16):
    """w [N, K] -> (float8_e4m3fn [N, K], scales [N]): scales[n] = max|w[n]| / 448 rounded to
    scale_dtype (1 for a row of zeros), stored row = w[n] / scales[n] rounded to e4m3."""
    amax = w.float().abs().amax(dim=1)
    scales = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax)).to(scale_dtype)
    q = (w.float() / scales.float()[:, None]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, scales


class WeightOnlyFp8Linear(nn.Module):
    """Drop-in for nn.Linear(bias=False): buffers `weight` [out, in] float8_e4m3fn and `scales` [out]."""

    def __init__(self, in_features: int, out_features: int, device=None, dtype=torch.bfloat16):
        super().__init__()
        assert in_features % 16 == 0, "the fp8 GEMV reads 16 weights per lane"
        self.in_features, self.out_features = in_features, out_features
        self.register_buffer("weight", torch.zeros(out_features, in_features, dtype=torch.float8_e4m3fn, device=device))
        self.register_buffer("scales", torch.ones(out_features, dtype=dtype, device=device))

    @classmethod
    def from_linear(cls, lin: nn.Linear) -> "WeightOnlyFp8Linear":
        assert lin.bias is None
        q = cls(lin.in_features, lin.out_features, device=lin.weight.device, dtype=lin.weight.dtype)
        w8, sc = quantize_fp8_rowwise(lin.weight.detach(), lin.weight.dtype)
        q.weight.copy_(w8)
        q.scales.copy_(sc)
        return q

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x = x.contiguous()
        return _hip.linear_fp8(x, self.weight, self.scales, x.new_empty(*x.shape[:-1], self.out_features))

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, weight=float8_e4m3fn"


def quantize_model_fp8(model: nn.Module, include_output: bool = True) -> nn.Module:
    """Replace every projection of the blocks (wqkv / wqkv1, wo, w1, w2) and, optionally, the lm_head by its
    weight-only fp8 form, in place.  Norm gains and the embedding table keep the model dtype."""
    for blk in model.layers:
        for parent in (getattr(blk, "attention", None), getattr(blk, "feed_forward", None)):
            if parent is None:
                continue
            for name, child in list(parent.named_children()):
                if isinstance(child, nn.Linear):
                    setattr(parent, name, WeightOnlyFp8Linear.from_linear(child))
    if include_output and isinstance(model.output, nn.Linear):
        model.output = WeightOnlyFp8Linear.from_linear(model.output)
    if hasattr(model, "_fused"):
        model._fused = {}
    return model
