"""RMSNorm with optional fused residual add, backed by gfx950 HIP kernels.

Drop-in for the reference's live ``RMSNorm`` (nanovllm/layers/layernorm.py:60-100):
``RMSNorm(hidden_size, eps=1e-6, dtype=None, device=None)`` with a ``weight`` parameter, and
``forward(x, residual=None)`` returning ``y`` or ``(y, new_residual)``.  Arithmetic is fp32
with ONE rounding to bf16 after the weight multiply (what the reference's compiled forward
produces); ``new_residual = bf16(f32(x) + f32(residual))``.  Inputs are never modified.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6, dtype: torch.dtype | None = None,
                 device: torch.device | None = None):
        super().__init__()
        self.hidden_size = hidden_size
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype, device=device))

    def forward(self, x: torch.Tensor, residual: torch.Tensor | None = None):
        if x.shape[-1] != self.hidden_size:
            raise ValueError(f"last dim {x.shape[-1]} != hidden_size {self.hidden_size}")
        if residual is None:
            return ops.rmsnorm(x, self.weight, self.eps)
        return ops.add_rmsnorm(x, residual, self.weight, self.eps)


class LayerNorm(nn.Module):
    """LayerNorm with weight and bias over an fp32 residual stream (float32 parameters): (x - mean) /
    sqrt(var + eps) * w + b, biased variance.  `forward(x)` normalises a float32 [T, W] tensor into `out_dtype`;
    `residual_boundary` below runs a post-norm, the stream update and the next pre-norm in one launch."""

    def __init__(self, hidden_size: int, eps: float = 1e-5, device: torch.device | None = None):
        super().__init__()
        self.hidden_size, self.eps = hidden_size, eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=torch.float32, device=device))
        self.bias = nn.Parameter(torch.zeros(hidden_size, dtype=torch.float32, device=device))

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        return ops.add_layernorm(x, pre=(self.weight, self.bias), out_dtype=out_dtype, eps=self.eps)


def residual_boundary(resid: torch.Tensor, h: torch.Tensor | None = None, post: LayerNorm | None = None,
                      extra: torch.Tensor | None = None, pre: LayerNorm | None = None,
                      out_dtype: torch.dtype = torch.float32):
    """In place on the float32 stream: resid += post(h) + extra (each part optional); returns pre(resid) in
    `out_dtype` (None without `pre`)."""
    eps = (post or pre).eps if (post or pre) is not None else 0.0
    return ops.add_layernorm(resid, h, (post.weight, post.bias) if post is not None else None, extra,
                             (pre.weight, pre.bias) if pre is not None else None, out_dtype, eps)
