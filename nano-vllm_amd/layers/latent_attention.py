"""Causal attention over a paged LATENT cache, backed by gfx950 HIP kernels.

Keys and values of a token are cached as one RMS-normed low-rank latent c [rank] plus one rotated key part k_r [R] that
all heads share.  With the key up-projection moved to the query (q_lat = Uk_h^T q_plain, done by the caller) and the
value up-projection moved behind the attention, this is multi-query attention with key [c | k_r] and value c:

  * ``nv_latent_prep_store``    normalises c, rotates k_r and the queries' rotated part, scatters the cache rows,
  * ``nv_attn_scoremod_paged``  the framework's paged attention with free head sizes (one kv head, fp32 softmax).

Rotary: pair i is turned by position * freq[i]; the pairing is (2i, 2i+1) or (i, i + R/2).  The frequencies are
base^(-2i/R), optionally blended for long contexts: with dim(t) = R ln(original / (2 pi t)) / (2 ln base),
lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), R - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
the frequency becomes f_i / factor * ramp_i + f_i (1 - ramp_i), and cos and sin are multiplied by 0.1 ln(factor) + 1.
The module owns no cache (a layer that runs several times per forward has one per run).
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import ops
from ..utils.cache_context import get_context


def blended_frequencies(dims: int, base: float, scaling: dict | None) -> tuple[torch.Tensor, float]:
    """(frequencies [dims / 2] float32 computed in double precision and rounded once, magnitude of cos / sin)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    mag = 1.0
    if scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def pair_of(turns: float) -> float:
            return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32), mag


class LatentAttention(nn.Module):
    def __init__(self, num_heads: int, rank: int, rot_dim: int, scale: float, eps: float, rot_base: float = 10000.0,
                 rot_scaling: dict | None = None, interleaved: bool = True, device=None):
        super().__init__()
        self.num_heads, self.rank, self.rot_dim = num_heads, rank, rot_dim
        self.scale, self.eps, self.interleaved = float(scale), eps, interleaved
        self.latent_norm = nn.Parameter(torch.ones(rank, dtype=torch.float32, device=device))
        freq, self.mag = blended_frequencies(rot_dim, rot_base, rot_scaling)
        self.register_buffer("freq", freq.to(device) if device is not None else freq, persistent=False)

    def forward(self, q: torch.Tensor, q_lat: torch.Tensor, ckv: torch.Tensor, positions: torch.Tensor,
                k_cache: torch.Tensor, v_cache: torch.Tensor) -> torch.Tensor:
        """q [T, H, Dq] (its last R columns get the rotary); q_lat [T, H, rank]; ckv [T, rank + R] as projected;
        k_cache [num_blocks, block_size, 1, rank + R]; v_cache [.., 1, rank]: a cache of its own, or the first `rank`
        columns of k_cache (then nothing is stored twice).  Returns [T, H, rank]."""
        ctx = get_context()
        q_full = ops.latent_prep_store(q, q_lat, ckv, self.latent_norm, self.freq, self.mag, self.interleaved, positions,
                                       ctx.slot_mapping, k_cache, v_cache, self.rot_dim, self.eps)
        singles = -1 if ctx.num_decode_seqs is None else int(ctx.num_decode_seqs > 0)
        o = ops.attn_scoremod_paged(q_full, k_cache, v_cache, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables,
                                    self.scale, 0.0, None, None, ctx.max_seqlen_q, ctx.max_seqlen_k, singles)
        return o.view(q.shape[0], self.num_heads, self.rank)
