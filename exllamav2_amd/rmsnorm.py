"""ExLlamaV2RMSNorm (reference rmsnorm.py:115-211)."""
from __future__ import annotations

import torch


class ExLlamaV2RMSNorm:
    def __init__(self, ext, key: str, weight: torch.Tensor, eps: float):
        self.ext = ext
        self.key = key
        self.weight = weight
        self.variance_epsilon = eps

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """rmsnorm.py:128-150 -> ext_c.rms_norm"""
        out = torch.empty_like(hidden_states)
        d = hidden_states.shape[-1]
        self.ext.rms_norm(hidden_states.view(-1, d), self.weight, out.view(-1, d), self.variance_epsilon)
        return out

    def forward_torch(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """rmsnorm.py:187-211 (fp32 torch reference path)"""
        variance = hidden_states.to(torch.float32).pow(2).mean(-1, keepdim=True)
        hidden_states = hidden_states * torch.rsqrt(variance + self.variance_epsilon)
        hidden_states = hidden_states.to(self.weight.dtype)
        return hidden_states * self.weight


class PostNorm:
    """The residual step of a post-norm layer, x <- rms_norm(alpha x + sublayer(x)) (1 + w), as ONE launch in place on the fp32
    residual stream (csrc/rowops.hip: post_norm_kernel); it also leaves the operand-dtype copy the next linears read.  The weight is
    stored around zero.  `moe` routes the mixture of a token's chosen experts (identity experts included) through the same launch."""

    def __init__(self, ext, key: str, weight: torch.Tensor, eps: float, alpha: float):
        self.ext, self.key, self.weight, self.eps, self.alpha = ext, key, weight.contiguous(), eps, alpha

    def forward(self, x32: torch.Tensor, xh, y, rows: int, moe=None) -> None:
        self.ext.post_norm(x32, xh, y, self.weight, rows, self.alpha, self.eps, moe=moe)


class PreLayerNorm:
    """The norm in front of a sublayer of a pre-norm layer: (x - mean) / sqrt(var + eps) * w + b.  It runs fused with the residual
    addition of the sublayer BEFORE it (csrc/rowops.hip: add_layer_norm_kernel): `forward` adds `y` (that sublayer's fp32 output, or
    None at the start of the stack) into the fp32 stream and leaves the normalised rows in the operand dtype."""

    def __init__(self, ext, key: str, weight: torch.Tensor, bias: torch.Tensor | None, eps: float):
        self.ext, self.key, self.weight, self.eps = ext, key, weight.contiguous(), eps
        self.bias = bias.contiguous() if bias is not None else None
        if self.bias is not None and self.bias.shape != self.weight.shape:
            raise RuntimeError(f"{key}: weight and bias differ in shape")

    def forward(self, x32: torch.Tensor, y, out: torch.Tensor, rows: int, row_idx=None) -> None:
        self.ext.add_layer_norm(x32, y, self.weight, self.bias, out, rows, self.eps, row_idx=row_idx)
