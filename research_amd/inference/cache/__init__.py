"""Host-side block allocators behind one protocol (reference: rollouts/rollouts/inference/cache/__init__.py).

``PagedKVCache`` is the reference's hash allocator restated, ``CountingPagedKVCache`` the same with growth by
token count, ``RadixKVCache`` the prefix tree that the reference only declares.  None of them owns device memory:
they hand out block ids, and the attention backend owns the pool those ids index.
"""

from .paged import Block, CountingPagedKVCache, PagedKVCache, compute_block_hash
from .protocol import KVCacheManager
from .radix import RadixKVCache

_ALLOCATORS = ("CountingPagedKVCache", "PagedKVCache", "RadixKVCache")
_PARTS = ("Block", "KVCacheManager", "compute_block_hash")
__all__ = [*_ALLOCATORS, *_PARTS]
