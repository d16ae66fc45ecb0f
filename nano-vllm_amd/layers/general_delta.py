"""Generalized delta rule with per-sequence state slots, backed by a gfx950 HIP kernel.

Per head a state S [D, D] (key channel x value channel) in float32 in ``state[slot]``:
S <- diag(w) S - (a * u)(u^T S) + k v^T, both terms reading the old state, with u the unit key,
w = exp(-decay_rate * sigmoid(w_raw + w_bias)) a decay and a = sigmoid(a_raw + a_bias) a removal rate per key channel;
the read-out S^T r is divided by its root mean square per head, weighted, and gated by sigmoid(gate_raw).
A sequence whose rows start at position 0 starts from zero whatever its slot held before.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import ops
from ..utils.cache_context import get_context


class GeneralDeltaRule(nn.Module):
    def __init__(self, num_heads: int, head_dim: int, eps: float, decay_rate: float = math.exp(-0.5),
                 key_eps: float = 1e-6, device=None):
        super().__init__()
        self.num_heads, self.head_dim, self.eps = num_heads, head_dim, eps
        self.decay_rate, self.key_eps = decay_rate, key_eps
        f32 = dict(dtype=torch.float32, device=device)
        self.a_bias = nn.Parameter(torch.zeros(num_heads * head_dim, **f32))
        self.w_bias = nn.Parameter(torch.zeros(num_heads * head_dim, **f32))
        self.norm_weight = nn.Parameter(torch.ones(num_heads * head_dim, **f32))

    def forward(self, r, k, v, w_raw, a_raw, gate_raw, state: torch.Tensor) -> torch.Tensor:
        """r, k, v: [T, H, D]; w_raw, a_raw, gate_raw: [T, H * D] as projected; state [slots, H, D, D] float32.
        Returns [T, H * D]."""
        ctx = get_context()
        return ops.general_delta_rule(r, k, v, w_raw, a_raw, gate_raw, self.w_bias, self.a_bias, self.norm_weight, state,
                                      ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.state_slots, self.eps, self.decay_rate,
                                      self.key_eps)
