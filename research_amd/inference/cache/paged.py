"""Host-side block allocator with hash-chained prefix reuse.

Behavioural twin of the reference allocator
(rollouts/rollouts/inference/cache/paged.py:57-230).  It owns no device
memory: it hands out integer block ids, and the block tables built from them
are what the attention kernels consume.  Sequences whose leading *full* blocks
hold equal tokens receive the same block ids, which is how several block
tables come to share prefix blocks.

The twin keeps the reference's observable quirks instead of repairing them,
because callers written against the reference see them:

* ``append_token`` grows a sequence only when its last block carries a hash,
  i.e. was filled completely by ``allocate`` (paged.py:194-201).  A partly
  filled last block never triggers growth, however many tokens are appended.
* Re-using a *freed* block on a prefix hit clears that block's hash and token
  record (paged.py:217-224 via :31-35), so it cannot be hit a second time.
* ``hash_to_block_id`` is never pruned when blocks are freed (paged.py:226-230).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Set, Tuple

import numpy as np
import xxhash

_NO_HASH = -1


@dataclass
class Block:
    """One pool block as the allocator sees it (paged.py:17-35)."""

    block_id: int
    ref_count: int = 0
    hash: int = _NO_HASH
    token_ids: list = field(default_factory=list)

    def update(self, hash: int, token_ids: list) -> None:
        self.hash, self.token_ids = hash, token_ids

    def reset(self) -> None:
        self.ref_count, self.hash, self.token_ids = 1, _NO_HASH, []


def compute_block_hash(token_ids: List[int], prefix_hash: int = _NO_HASH) -> int:
    """xxh64 over ``[previous block's hash as 8 LE bytes] ++ token bytes``.

    Layout from paged.py:38-54: the tokens are serialised the way
    ``numpy.array(list_of_int).tobytes()`` does (native int64, little endian
    on this platform); the first block of a chain has no prefix bytes.
    """
    state = xxhash.xxh64()
    if prefix_hash != _NO_HASH:
        state.update(int(prefix_hash).to_bytes(8, "little"))
    state.update(np.array(token_ids).tobytes())
    return state.intdigest()


class PagedKVCache:
    def __init__(self, num_blocks: int, block_size: int = 16) -> None:
        assert num_blocks > 0
        assert block_size > 0
        self.block_size = block_size
        self.blocks: List[Block] = [Block(b) for b in range(num_blocks)]
        self.hash_to_block_id: Dict[int, int] = {}
        self.free_block_ids: Deque[int] = deque(range(num_blocks))
        self.used_block_ids: Set[int] = set()
        self.seq_to_blocks: Dict[int, List[int]] = {}
        self.seq_cached_tokens: Dict[int, int] = {}

    # -- queries ---------------------------------------------------------
    def num_free_blocks(self) -> int:
        return len(self.free_block_ids)

    def _blocks_for(self, num_tokens: int) -> int:
        return -(-num_tokens // self.block_size)

    def can_allocate(self, num_tokens: int) -> bool:
        return self._blocks_for(num_tokens) <= len(self.free_block_ids)

    def get_block_ids(self, seq_id: int) -> Tuple[int, ...]:
        return tuple(self.seq_to_blocks.get(seq_id, ()))

    def get_cached_tokens(self, seq_id: int) -> int:
        return self.seq_cached_tokens.get(seq_id, 0)

    # -- lifecycle -------------------------------------------------------
    def allocate(self, seq_id: int, token_ids: List[int]) -> Tuple[int, ...]:
        """Give ``seq_id`` blocks for ``token_ids`` (paged.py:97-163).

        Leading full blocks are looked up by chained hash until the first
        miss; everything after the first miss (and the trailing partial block)
        is taken from the head of the free queue.
        """
        assert seq_id not in self.seq_to_blocks, f"Sequence {seq_id} already allocated"
        bs = self.block_size
        n_blocks = self._blocks_for(len(token_ids))
        chunks = [token_ids[i * bs : (i + 1) * bs] for i in range(n_blocks)]

        owned: List[int] = []
        chain = _NO_HASH
        hits = 0
        probing = True
        for toks in chunks:
            full = len(toks) == bs
            digest = compute_block_hash(toks, chain) if full else _NO_HASH
            if full and probing:
                candidate = self.hash_to_block_id.get(digest, -1)
                if candidate != -1 and self.blocks[candidate].token_ids == toks:
                    if candidate in self.used_block_ids:
                        self.blocks[candidate].ref_count += 1
                    else:
                        # revived from the free queue: _take() wipes its record
                        self._take(candidate)
                    owned.append(candidate)
                    hits += 1
                    chain = digest
                    continue
                probing = False
            fresh = self.free_block_ids[0]
            blk = self._take(fresh)
            owned.append(fresh)
            if full:
                blk.update(digest, toks)
                self.hash_to_block_id[digest] = fresh
                chain = digest

        self.seq_to_blocks[seq_id] = owned
        self.seq_cached_tokens[seq_id] = hits * bs
        return tuple(owned)

    def deallocate(self, seq_id: int) -> None:
        """Drop one reference from each block, last block first (paged.py:165-177)."""
        owned = self.seq_to_blocks.get(seq_id)
        if owned is None:
            return
        for block_id in owned[::-1]:
            blk = self.blocks[block_id]
            blk.ref_count -= 1
            if blk.ref_count == 0:
                self._release(block_id)
        del self.seq_to_blocks[seq_id]
        del self.seq_cached_tokens[seq_id]

    def append_token(self, seq_id: int, token_id: int) -> Optional[int]:
        """Grow by one block iff the last block is hash-complete (paged.py:179-203)."""
        assert seq_id in self.seq_to_blocks
        owned = self.seq_to_blocks[seq_id]
        if self.blocks[owned[-1]].hash == _NO_HASH:
            return None
        if not self.free_block_ids:
            raise RuntimeError("No free blocks for token append")
        fresh = self.free_block_ids[0]
        self._take(fresh)
        owned.append(fresh)
        return fresh

    # -- internals -------------------------------------------------------
    def _take(self, block_id: int) -> Block:
        blk = self.blocks[block_id]
        assert blk.ref_count == 0, f"Block {block_id} already in use"
        blk.reset()
        self.free_block_ids.remove(block_id)
        self.used_block_ids.add(block_id)
        return blk

    def _release(self, block_id: int) -> None:
        assert self.blocks[block_id].ref_count == 0
        self.used_block_ids.remove(block_id)
        self.free_block_ids.append(block_id)

    # names the reference uses for the two internals (paged.py:217, :226)
    _allocate_block = _take
    _deallocate_block = _release


class CountingPagedKVCache(PagedKVCache):
    """``PagedKVCache`` that grows by token count.

    The reference's ``append_token`` hands out a block only when the last block was filled completely by
    ``allocate`` (paged.py:194-201), so a sequence whose prompt is not a whole number of blocks never grows.
    An engine that decodes past the first block boundary needs growth exactly when a token starts a new block;
    this subclass counts tokens and does that, and leaves allocation, prefix reuse and release as they are.
    """

    def __init__(self, num_blocks: int, block_size: int = 16) -> None:
        super().__init__(num_blocks, block_size)
        self.seq_num_tokens: Dict[int, int] = {}

    def blocks_needed(self, token_ids: List[int]) -> int:
        """Blocks ``allocate(token_ids)`` would take from the free queue: every block of the prompt except the
        leading ones found cached in blocks that some sequence still holds (a cached block nobody holds sits in
        the free queue and is taken from there)."""
        bs = self.block_size
        n_blocks = self._blocks_for(len(token_ids))
        chain = _NO_HASH
        shared = 0
        for i in range(len(token_ids) // bs):
            toks = token_ids[i * bs : (i + 1) * bs]
            chain = compute_block_hash(toks, chain)
            candidate = self.hash_to_block_id.get(chain, -1)
            if candidate == -1 or self.blocks[candidate].token_ids != toks:
                break
            if candidate in self.used_block_ids:
                shared += 1
        return n_blocks - shared

    def allocate(self, seq_id: int, token_ids: List[int]) -> Tuple[int, ...]:
        """All or nothing: the reference's ``allocate`` runs out of blocks half-way (``IndexError`` from the
        empty free queue, paged.py:150) and leaves the blocks it had taken owned by nobody; here the need is
        checked first and a call that cannot be served raises before anything changes."""
        need = self.blocks_needed(token_ids)
        if need > len(self.free_block_ids):
            raise RuntimeError(f"No free blocks for sequence {seq_id}: needs {need}, "
                               f"{len(self.free_block_ids)} free")
        blocks = super().allocate(seq_id, token_ids)
        self.seq_num_tokens[seq_id] = len(token_ids)
        return blocks

    def deallocate(self, seq_id: int) -> None:
        super().deallocate(seq_id)
        self.seq_num_tokens.pop(seq_id, None)

    def append_token(self, seq_id: int, token_id: int) -> Optional[int]:
        assert seq_id in self.seq_to_blocks
        n = self.seq_num_tokens[seq_id]
        fresh = None
        if n % self.block_size == 0:
            if not self.free_block_ids:
                raise RuntimeError("No free blocks for token append")
            fresh = self.free_block_ids[0]
            self._take(fresh)
            self.seq_to_blocks[seq_id].append(fresh)
        self.seq_num_tokens[seq_id] = n + 1
        return fresh
