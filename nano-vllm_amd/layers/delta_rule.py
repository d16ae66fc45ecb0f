"""Recurrent mixer layers with per-sequence state slots, backed by gfx950 HIP kernels.

``ShortConvSilu``: a short causal convolution over time per channel followed by SiLU; the last taps-1 inputs of each
sequence are carried in ``conv_state[slot]``.  ``GatedDeltaRule``: the delta rule S <- diag(g) S + k (beta (v - S^T
k))^T with one decay per head and key channel, unit-norm q / k, and a normalised, gated read-out; the state
[H, D, Dv] of each sequence lives in float32 in ``state[slot]``.

A slot is a row of the state tensors.  The engine gives a request a slot at admission and takes it back when the
request ends; the step's ``CacheContext.state_slots`` names the slot of every sequence of the batch.  A sequence
whose rows start at position 0 starts from zero whatever its slot held before, so slots need no clearing.
The modules own no state: a layer that runs several times per forward has one state per run, passed in.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..utils.cache_context import get_context


class ShortConvSilu(nn.Module):
    def __init__(self, channels: int, taps: int, device=None):
        super().__init__()
        self.channels, self.taps = channels, taps
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32, device=device))

    def forward(self, x: torch.Tensor, conv_state: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        return ops.causal_conv_silu(x, self.weight, conv_state, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.state_slots)


class GatedDeltaRule(nn.Module):
    def __init__(self, num_heads: int, num_qk_heads: int, head_dim: int, v_head_dim: int, eps: float, device=None):
        super().__init__()
        assert num_heads % num_qk_heads == 0
        self.num_heads, self.num_qk_heads, self.head_dim, self.v_head_dim, self.eps = \
            num_heads, num_qk_heads, head_dim, v_head_dim, eps
        f32 = dict(dtype=torch.float32, device=device)
        self.A_log = nn.Parameter(torch.zeros(num_heads, **f32))
        self.dt_bias = nn.Parameter(torch.zeros(num_heads * head_dim, **f32))
        self.norm_weight = nn.Parameter(torch.ones(v_head_dim, **f32))

    def forward(self, q, k, v, a_raw, b_raw, gate_raw, state: torch.Tensor) -> torch.Tensor:
        """q, k: [T, G, D]; v: [T, H, Dv] (after the short convolution); a_raw [T, H*D], b_raw [T, H],
        gate_raw [T, H*Dv] as projected; state [slots, H, D, Dv] float32.  Returns [T, H*Dv]."""
        ctx = get_context()
        return ops.gated_delta_rule(q, k, v, a_raw, b_raw, gate_raw, self.A_log, self.dt_bias, self.norm_weight, state,
                                    ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.state_slots, self.eps)
