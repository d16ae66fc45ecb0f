"""Routed experts (mixture of experts), backed by gfx950 HIP kernels: top-k routing with a softmax over the chosen
logits, the (token, choice) pairs sorted by expert on the device, and both expert products as grouped MFMA matrix
products over row tiles of one expert each (no host round trip, no atomics).

Expert: g = min(G h, limit), u = clamp(U h, -limit, limit), D (g * sigmoid(alpha g) * (u + 1)); no biases.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops


class MoEExperts(nn.Module):
    def __init__(self, top: int, limit: float, alpha: float = 1.702):
        super().__init__()
        self.top, self.limit, self.alpha = int(top), float(limit), float(alpha)

    def forward(self, h: torch.Tensor, logits: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
        """h [T, W]; logits [T, E] float32; gate_up [E, 2 ff, W] (gate rows, then up rows); down [E, W, ff].
        Returns the weighted expert outputs [T, top, W] float32."""
        return ops.moe_experts(h, logits, gate_up, down, self.top, self.limit, self.alpha)
