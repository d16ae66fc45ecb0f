"""What a model asks of the runner's cache and state manager, one entry per cache the forward pass uses
(a layer that runs several times with shared weights asks for one per run).

PagedKVSpec: a paged KV cache k [num_blocks, block_size, kv_heads, key_dim], v [.., kv_heads, value_dim] addressed
through the step's block tables and slot mapping (all paged caches of a model share the block numbering).  With
`value_in_key` the value of a token IS the first value_dim columns of its key row (a cached latent that serves as both):
nothing is allocated for v, the layer gets the column range of k as its value cache.
SlotStateSpec: named per-sequence state tensors [num_state_slots, *shape]; the sequence's row is
`CacheContext.state_slots[b]`.  dtype None = the model's compute dtype.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch


@dataclass
class PagedKVSpec:
    kv_heads: int
    key_dim: int
    value_dim: int
    value_in_key: bool = False

    def block_elems(self, block_size: int) -> int:
        return block_size * self.kv_heads * (self.key_dim + (0 if self.value_in_key else self.value_dim))


@dataclass
class SlotStateSpec:
    tensors: dict = field(default_factory=dict)      # name -> (shape per slot, dtype or None)

    def slot_bytes(self, dtype: torch.dtype) -> int:
        total = 0
        for shape, dt in self.tensors.values():
            n = 1
            for s in shape:
                n *= s
            total += n * (dt or dtype).itemsize
        return total
