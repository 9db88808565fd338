"""Host-side block allocators (reference: rollouts/rollouts/inference/cache/__init__.py)."""

from .paged import Block, CountingPagedKVCache, PagedKVCache, compute_block_hash
from .protocol import KVCacheManager
from .radix import RadixKVCache

__all__ = ["PagedKVCache", "CountingPagedKVCache", "RadixKVCache", "Block", "KVCacheManager", "compute_block_hash"]
