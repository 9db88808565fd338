"""Prefix-tree block allocator behind the ``KVCacheManager`` protocol.

The reference declares this allocator but ships only a stub whose constructor
raises (rollouts/rollouts/inference/cache/radix.py:15-61; the protocol it is
meant to satisfy is cache/protocol.py:9-43).  This is an implementation of what
that stub describes: N rollouts of one prompt walk the same path of the tree
and receive the same block ids, so their block tables share the prefix blocks
and the attention kernels read them once per sharer from cache rather than N
private copies.  Like ``PagedKVCache`` it owns no device memory.

Design (block-granular radix tree):

* A node is one *full* block of tokens; the edge from its parent is keyed by
  those ``block_size`` token ids, so a path from the root spells a prefix in
  whole blocks and lookup is exact (no hashes, no collisions).
* ``allocate`` walks the tree as far as the prompt's full blocks match
  (``get_cached_tokens`` = matched blocks x block_size), takes a reference on
  every node on the way, creates nodes for the remaining full blocks and one
  private block for a trailing partial block.
* ``append_token`` counts tokens: a new block is handed out exactly when the
  token lands in a block the sequence does not have yet; a private block that
  fills up is entered into the tree (unless an equal node already exists, in
  which case the sequence keeps its private copy).
* ``deallocate`` drops the references.  Nodes nobody references stay in the
  tree as cached prefixes and count as free capacity; when the free list runs
  dry they are evicted least-recently-used first, leaves before their parents
  (a node is referenced by every sequence that references a descendant, so an
  unreferenced node only has unreferenced descendants).
"""

from __future__ import annotations

from collections import OrderedDict, deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Tuple


@dataclass
class RadixNode:
    """One full block in the tree (fields as the reference's stub names them, radix.py:16-23)."""

    token_ids: Tuple[int, ...]  # the block's tokens = the key of the edge from the parent
    block_id: int
    children: Dict[Tuple[int, ...], "RadixNode"] = field(default_factory=dict)
    ref_count: int = 0
    parent: Optional["RadixNode"] = None


@dataclass
class _Sequence:
    path: List[RadixNode]        # tree nodes of the leading full blocks
    private: List[int]           # block ids after the path (not in the tree)
    tail_tokens: List[int]       # tokens held by the private blocks
    cached_tokens: int
    num_tokens: int


class RadixKVCache:
    def __init__(self, num_blocks: int, block_size: int = 16) -> None:
        assert num_blocks > 0
        assert block_size > 0
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.root = RadixNode(token_ids=(), block_id=-1)
        self.free_block_ids: Deque[int] = deque(range(num_blocks))
        # unreferenced nodes, least recently used first
        self._idle: "OrderedDict[int, RadixNode]" = OrderedDict()
        self._seqs: Dict[int, _Sequence] = {}

    # -- queries ---------------------------------------------------------
    def num_free_blocks(self) -> int:
        """Blocks that an allocation could obtain: never-used or released ones plus cached, unreferenced ones."""
        return len(self.free_block_ids) + len(self._idle)

    def _blocks_for(self, num_tokens: int) -> int:
        return -(-num_tokens // self.block_size)

    def can_allocate(self, num_tokens: int) -> bool:
        """Conservative: ignores any prefix the tokens might share with the tree."""
        return self._blocks_for(num_tokens) <= self.num_free_blocks()

    def get_block_ids(self, seq_id: int) -> Tuple[int, ...]:
        seq = self._seqs.get(seq_id)
        if seq is None:
            return ()
        return tuple(node.block_id for node in seq.path) + tuple(seq.private)

    def get_cached_tokens(self, seq_id: int) -> int:
        seq = self._seqs.get(seq_id)
        return seq.cached_tokens if seq is not None else 0

    def match_prefix(self, token_ids: List[int]) -> int:
        """Number of leading tokens of ``token_ids`` that the tree holds (whole blocks); changes nothing."""
        node, n = self.root, 0
        bs = self.block_size
        for i in range(len(token_ids) // bs):
            node = node.children.get(tuple(token_ids[i * bs : (i + 1) * bs]))
            if node is None:
                break
            n += bs
        return n

    # -- lifecycle -------------------------------------------------------
    def allocate(self, seq_id: int, token_ids: List[int]) -> Tuple[int, ...]:
        assert seq_id not in self._seqs, f"Sequence {seq_id} already allocated"
        bs = self.block_size
        n_full = len(token_ids) // bs
        chunks = [tuple(token_ids[i * bs : (i + 1) * bs]) for i in range(n_full)]
        # walk the matching prefix first and pin it, so that eviction below cannot take it
        path: List[RadixNode] = []
        node = self.root
        for toks in chunks:
            child = node.children.get(toks)
            if child is None:
                break
            self._ref(child)
            path.append(child)
            node = child
        hits = len(path)
        need = (n_full - hits) + (1 if len(token_ids) % bs else 0)
        have = self.num_free_blocks()
        if need > have:
            for pinned in reversed(path):
                self._unref(pinned)
            raise RuntimeError(f"No free blocks: need {need} beyond the cached prefix, have {have}")
        for toks in chunks[hits:]:
            child = RadixNode(token_ids=toks, block_id=self._take_block(), parent=node)
            node.children[toks] = child
            self._ref(child)
            path.append(child)
            node = child
        private: List[int] = []
        tail = list(token_ids[n_full * bs :])
        if tail:
            private.append(self._take_block())
        self._seqs[seq_id] = _Sequence(path=path, private=private, tail_tokens=tail, cached_tokens=hits * bs,
                                       num_tokens=len(token_ids))
        return self.get_block_ids(seq_id)

    def deallocate(self, seq_id: int) -> None:
        seq = self._seqs.pop(seq_id, None)
        if seq is None:
            return
        for block_id in reversed(seq.private):
            self.free_block_ids.append(block_id)
        for node in reversed(seq.path):  # leaves become idle (and so evictable) before their parents
            self._unref(node)

    def append_token(self, seq_id: int, token_id: int) -> Optional[int]:
        """Record one more token; returns the new block id when the token starts a new block, else None."""
        assert seq_id in self._seqs
        seq = self._seqs[seq_id]
        bs = self.block_size
        fresh = None
        if seq.num_tokens % bs == 0:  # every block the sequence has is full
            if self.num_free_blocks() == 0:
                raise RuntimeError("No free blocks for token append")
            fresh = self._take_block()
            seq.private.append(fresh)
        seq.tail_tokens.append(token_id)
        seq.num_tokens += 1
        # a private block that follows the tree path directly and is now full joins the tree
        if len(seq.private) == 1 and len(seq.tail_tokens) == bs:
            parent = seq.path[-1] if seq.path else self.root
            toks = tuple(seq.tail_tokens)
            if toks not in parent.children:
                node = RadixNode(token_ids=toks, block_id=seq.private[0], parent=parent, ref_count=1)
                parent.children[toks] = node
                seq.path.append(node)
                seq.private.clear()
                seq.tail_tokens.clear()
        # (blocks behind a private copy stay private: their prefix is not a tree path)
        return fresh

    # -- internals -------------------------------------------------------
    def _ref(self, node: RadixNode) -> None:
        if node.ref_count == 0:
            self._idle.pop(node.block_id, None)
        node.ref_count += 1

    def _unref(self, node: RadixNode) -> None:
        assert node.ref_count > 0
        node.ref_count -= 1
        if node.ref_count == 0:
            self._idle[node.block_id] = node  # most recently used end

    def _take_block(self) -> int:
        if self.free_block_ids:
            return self.free_block_ids.popleft()
        # evict the least recently used idle leaf
        for block_id, node in self._idle.items():
            if not node.children:
                del self._idle[block_id]
                del node.parent.children[node.token_ids]
                node.parent = None
                return block_id
        raise RuntimeError("No free blocks")
