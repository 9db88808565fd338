"""Interface of a host-side block allocator.

Method set of the reference's ``KVCacheManager``
(rollouts/rollouts/inference/cache/protocol.py:9-43).
"""

from __future__ import annotations

from typing import List, Optional, Protocol, Tuple


class KVCacheManager(Protocol):
    def num_free_blocks(self) -> int: ...

    def can_allocate(self, num_tokens: int) -> bool: ...

    def allocate(self, seq_id: int, token_ids: List[int]) -> Tuple[int, ...]: ...

    def deallocate(self, seq_id: int) -> None: ...

    def append_token(self, seq_id: int, token_id: int) -> Optional[int]: ...

    def get_block_ids(self, seq_id: int) -> Tuple[int, ...]: ...
