"""Pure functions from allocator state to an ``InferenceContext``.

Same names, arguments and results as the reference builders
(rollouts/rollouts/inference/context.py:10-154).  The slot of token position
``pos`` of a sequence with block ids ``blocks`` is

    blocks[pos // block_size] * block_size + pos % block_size

and ``-1`` when the table is too short to hold ``pos`` (context.py:35-42 and
:78-85); a ``-1`` slot makes the KV append drop that token's row.

``build_chunked_prefill_context`` is an addition: the reference has no chunked
prefill.  It numbers the chunk's tokens from ``prefix_len`` instead of from 0
and reduces to ``build_prefill_context`` when every prefix length is 0.
"""

from __future__ import annotations

from typing import List, Sequence, Tuple

from .cache.paged import PagedKVCache
from .types import InferenceContext


def _slot(blocks: Sequence[int], pos: int, block_size: int) -> int:
    idx, off = divmod(pos, block_size)
    return blocks[idx] * block_size + off if idx < len(blocks) else -1


def _ctx(is_prefill: bool, slots: List[int], seq_lens, block_tables, **extra) -> InferenceContext:
    return InferenceContext(
        is_prefill=is_prefill,
        slot_mapping=tuple(slots),
        block_tables=tuple(block_tables),
        seq_lens=tuple(seq_lens),
        max_seq_len=max(seq_lens) if seq_lens else 0,
        **extra,
    )


def build_prefill_context(
    cache: PagedKVCache,
    seq_ids: List[int],
    seq_lens: List[int],
    block_tables: List[Tuple[int, ...]],
) -> InferenceContext:
    """Slots for positions ``0..len-1`` of every sequence (context.py:10-50)."""
    bs = cache.block_size
    slots = [_slot(blocks, pos, bs) for n, blocks in zip(seq_lens, block_tables) for pos in range(n)]
    return _ctx(True, slots, seq_lens, block_tables)


def build_decode_context(
    cache: PagedKVCache,
    seq_ids: List[int],
    seq_lens: List[int],
    block_tables: List[Tuple[int, ...]],
) -> InferenceContext:
    """One slot per sequence, for position ``len-1`` (context.py:53-93).

    ``seq_lens`` already counts the token being appended in this step.
    """
    bs = cache.block_size
    slots = [_slot(blocks, n - 1, bs) for n, blocks in zip(seq_lens, block_tables)]
    return _ctx(False, slots, seq_lens, block_tables)


def build_chunked_prefill_context(
    cache: PagedKVCache,
    seq_ids: List[int],
    prefix_lens: List[int],
    chunk_lens: List[int],
    block_tables: List[Tuple[int, ...]],
) -> InferenceContext:
    """Prefill of ``chunk_lens[i]`` new tokens on top of ``prefix_lens[i]`` cached ones.

    ``seq_lens`` of the result is the total context (prefix + chunk);
    ``slot_mapping`` covers only the chunk's tokens.
    """
    bs = cache.block_size
    slots = [
        _slot(blocks, p + i, bs)
        for p, c, blocks in zip(prefix_lens, chunk_lens, block_tables)
        for i in range(c)
    ]
    totals = [p + c for p, c in zip(prefix_lens, chunk_lens)]
    return _ctx(True, slots, totals, block_tables, prefix_lens=tuple(prefix_lens))


def allocate_and_build_context(
    cache: PagedKVCache,
    seq_id: int,
    token_ids: List[int],
) -> Tuple[InferenceContext, int]:
    """``allocate`` then a single-sequence prefill context (context.py:96-123)."""
    blocks = cache.allocate(seq_id, token_ids)
    ctx = build_prefill_context(cache, [seq_id], [len(token_ids)], [blocks])
    return ctx, cache.get_cached_tokens(seq_id)


def extend_and_build_context(
    cache: PagedKVCache,
    seq_id: int,
    new_token: int,
    current_len: int,
) -> InferenceContext:
    """``append_token`` then a single-sequence decode context (context.py:126-154)."""
    cache.append_token(seq_id, new_token)
    return build_decode_context(cache, [seq_id], [current_len + 1], [cache.get_block_ids(seq_id)])
