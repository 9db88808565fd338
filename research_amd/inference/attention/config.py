"""Dimensions of the paged KV pool.

Same fields, defaults, derived properties and hashing rule as the reference's
``CacheConfig`` (rollouts/rollouts/inference/attention/config.py:8-58), plus
one optional field for the fp8-e4m3 pool layout this backend adds.
"""

from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class CacheConfig:
    num_layers: int
    num_kv_heads: int
    head_dim: int
    num_blocks: int = 1024
    block_size: int = 16
    sliding_window: Optional[int] = None
    dtype: torch.dtype = torch.bfloat16
    device: str = "cuda"
    # Extension: "fp8_e4m3" keeps K/V as one byte per element with one fp32
    # scale per (block, kv head); ``dtype`` then names the q / output type.
    kv_format: Optional[str] = None

    @property
    def total_slots(self) -> int:
        # config.py:38-40 of the reference
        return self.block_size * self.num_blocks

    @property
    def cache_shape(self) -> Tuple[int, int, int, int]:
        # config.py:43-45 of the reference: layer-major, then slot, head, dim
        return (self.num_layers, self.total_slots, self.num_kv_heads, self.head_dim)

    def __hash__(self) -> int:
        # torch dtypes are hashed through their name, as the reference does
        # (config.py:47-58); the extension field is appended only when set so
        # that reference-shaped configs hash to the reference's value.
        key = tuple(
            str(getattr(self, f.name)) if f.name == "dtype" else getattr(self, f.name)
            for f in fields(self)
            if f.name != "kv_format"
        )
        if self.kv_format is not None:
            key = key + (self.kv_format,)
        return hash(key)
