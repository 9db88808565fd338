"""Placeholder with the reference's behaviour: constructing it raises.

The reference ships only a stub for a prefix-tree allocator
(rollouts/rollouts/inference/cache/radix.py:26-61, ``__init__`` raises
``NotImplementedError`` at :43).  At the kernel boundary a prefix tree and the
hash-chained allocator in ``paged.py`` look the same: several block tables
name the same block ids.
"""

from __future__ import annotations


class RadixKVCache:
    def __init__(self, num_blocks: int, block_size: int = 16) -> None:
        raise NotImplementedError("RadixKVCache not yet implemented. Use PagedKVCache for now.")
