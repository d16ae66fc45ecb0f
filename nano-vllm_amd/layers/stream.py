"""Layers around an fp32 residual stream with one grouped RMS norm per layer, backed by gfx950 HIP kernels.

``stream_boundary``: everything that happens to the stream between two sublayers in ONE launch: the parallel
sublayers' outputs (a matmul-dtype tensor and / or fp32 parts such as the weighted outputs of routed experts) are added
times a multiplier, an RMS-normed side input is added times the same multiplier, the stream is handed on in the matmul
dtype, and / or the next layer's grouped RMS norm is taken (the row is cut into equal consecutive parts, each divided by
its own root mean square).  ``CausalConvAdd``: x + a short causal convolution of x over time per channel, the last taps-1
inputs of each sequence carried in float32 in ``state[slot]``.  ``TokenGate``: gelu_tanh(z) times a slice of a per-token
table row.  The modules own no state: a layer that runs several times per forward has one state per run, passed in.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..utils.cache_context import get_context

stream_boundary = ops.stream_boundary
rms_norm_rows = ops.rms_norm_rows


class CausalConvAdd(nn.Module):
    def __init__(self, channels: int, taps: int, device=None):
        super().__init__()
        self.channels, self.taps = channels, taps
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32, device=device))

    def forward(self, x: torch.Tensor, state: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        """x [T, C] float32; state [slots, taps - 1, C] float32; returns x + conv(x) in out_dtype."""
        ctx = get_context()
        return ops.causal_conv_add(x, self.weight, state, out_dtype, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.state_slots)


class TokenGate(nn.Module):
    """gelu_tanh(z) * table[ids, offset : offset + dim]."""

    def __init__(self, offset: int, dim: int):
        super().__init__()
        self.offset, self.dim = offset, dim

    def forward(self, z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        return ops.token_gate(z, table, ids, self.offset, self.dim)
