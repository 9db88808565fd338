"""Host-side allocator and context builders against the facts the reference's
own script asserts (rollouts/examples/inference/test_kv_cache.py:21-78) and
against scenarios traced by hand from rollouts/rollouts/inference/cache/paged.py."""

import struct

import numpy as np
import pytest
import xxhash

from research_amd.inference import (
    InferenceContext,
    PagedKVCache,
    allocate_and_build_context,
    build_chunked_prefill_context,
    build_decode_context,
    build_prefill_context,
    extend_and_build_context,
)
from research_amd.inference.cache import RadixKVCache, compute_block_hash


# ---- facts asserted by the reference's script ---------------------------------
def test_reference_allocate_deallocate_facts():
    cache = PagedKVCache(num_blocks=16, block_size=4)
    blocks = cache.allocate(seq_id=0, token_ids=[1, 2, 3, 4, 5, 6, 7])
    assert len(blocks) == 2  # test_kv_cache.py:28-31
    assert cache.num_free_blocks() == 14  # :32
    cache.deallocate(seq_id=0)
    assert cache.num_free_blocks() == 16  # :36-37


def test_reference_prefix_caching_fact():
    cache = PagedKVCache(num_blocks=16, block_size=4)
    toks = [1, 2, 3, 4, 5, 6, 7, 8]
    cache.allocate(seq_id=0, token_ids=toks)
    cache.allocate(seq_id=1, token_ids=toks + [9, 10])
    assert cache.get_cached_tokens(seq_id=1) == 8  # :41-46


def test_reference_context_builder_facts():
    cache = PagedKVCache(num_blocks=16, block_size=4)
    ctx, cached = allocate_and_build_context(cache, seq_id=0, token_ids=[1, 2, 3, 4, 5])
    assert ctx.is_prefill and len(ctx.slot_mapping) == 5  # :63-67
    assert cached == 0
    cache = PagedKVCache(num_blocks=16, block_size=4)
    cache.allocate(seq_id=0, token_ids=[1, 2, 3])
    ctx = extend_and_build_context(cache, seq_id=0, new_token=4, current_len=3)
    assert not ctx.is_prefill and len(ctx.slot_mapping) == 1  # :71-75


# ---- block hash ----------------------------------------------------------------
def test_xxh64_published_vector():
    # XXH64 of the empty input with seed 0, from the xxHash specification
    assert xxhash.xxh64(b"").intdigest() == 0xEF46DB3751D8E999


def test_block_hash_layout():
    toks = [5, 6, 7, 8]
    raw = struct.pack("<4q", *toks)  # int64 little endian, as numpy serialises a list of ints
    assert compute_block_hash(toks) == xxhash.xxh64(raw).intdigest()
    prev = compute_block_hash(toks)
    assert compute_block_hash([9, 9, 9, 9], prev) == xxhash.xxh64(
        prev.to_bytes(8, "little") + struct.pack("<4q", 9, 9, 9, 9)).intdigest()
    assert compute_block_hash(toks) != compute_block_hash(toks, prev)


# ---- allocator behaviour traced from paged.py ------------------------------------
def test_fifo_block_ids_and_shared_prefix_tables():
    cache = PagedKVCache(num_blocks=8, block_size=2)
    a = cache.allocate(0, [1, 2, 3, 4, 5])
    assert a == (0, 1, 2)
    b = cache.allocate(1, [1, 2, 3, 4, 9, 9, 7])
    # two full blocks shared, then fresh blocks from the head of the free queue
    assert b == (0, 1, 3, 4)
    assert cache.get_cached_tokens(1) == 4
    assert cache.blocks[0].ref_count == 2 and cache.blocks[1].ref_count == 2
    cache.deallocate(0)
    assert cache.num_free_blocks() == 4  # block 2 returned; 0 and 1 still held by seq 1
    assert list(cache.free_block_ids) == [5, 6, 7, 2]
    cache.deallocate(1)
    # freed last-block-first: 4, 3, 1, 0
    assert list(cache.free_block_ids) == [5, 6, 7, 2, 4, 3, 1, 0]
    cache.deallocate(1)  # unknown sequence: no-op
    assert cache.num_free_blocks() == 8


def test_lookup_stops_at_first_miss():
    cache = PagedKVCache(num_blocks=8, block_size=2)
    cache.allocate(0, [1, 2, 3, 4, 5, 6])
    got = cache.allocate(1, [1, 2, 7, 7, 5, 6])
    assert got[0] == 0 and got[1] != 1 and got[2] != 2
    assert cache.get_cached_tokens(1) == 2


def test_revived_block_loses_its_record():
    """paged.py:217-224 via :31-35: a hit on a freed block resets hash and tokens."""
    cache = PagedKVCache(num_blocks=4, block_size=2)
    cache.allocate(0, [1, 2])
    cache.deallocate(0)
    assert cache.allocate(1, [1, 2]) == (0,)  # hit on the freed block 0
    assert cache.get_cached_tokens(1) == 2
    assert cache.blocks[0].hash == -1 and cache.blocks[0].token_ids == []
    # the stale map entry still points at block 0, whose record is gone: miss
    assert cache.allocate(2, [1, 2]) == (1,)
    assert cache.get_cached_tokens(2) == 0
    assert cache.hash_to_block_id[compute_block_hash([1, 2])] == 1


def test_hash_map_is_never_pruned():
    cache = PagedKVCache(num_blocks=4, block_size=2)
    cache.allocate(0, [1, 2, 3, 4])
    cache.deallocate(0)
    assert len(cache.hash_to_block_id) == 2  # paged.py:226-230 leaves the map alone


def test_append_token_grows_only_after_a_hash_complete_block():
    cache = PagedKVCache(num_blocks=4, block_size=2)
    cache.allocate(0, [1, 2, 3])  # last block partial, no hash
    assert cache.append_token(0, 4) is None
    assert cache.append_token(0, 5) is None  # still no growth (paged.py:194-201)
    assert cache.get_block_ids(0) == (0, 1)
    cache.allocate(1, [7, 8])  # last block complete
    assert cache.append_token(1, 9) == 3
    assert cache.get_block_ids(1) == (2, 3)
    assert cache.append_token(1, 10) is None  # new last block has no hash
    with pytest.raises(AssertionError):
        cache.append_token(99, 1)


def test_append_token_without_free_blocks_raises():
    cache = PagedKVCache(num_blocks=1, block_size=2)
    cache.allocate(0, [1, 2])
    with pytest.raises(RuntimeError, match="No free blocks"):
        cache.append_token(0, 3)


def test_allocate_errors():
    cache = PagedKVCache(num_blocks=1, block_size=2)
    cache.allocate(0, [1])
    with pytest.raises(AssertionError):
        cache.allocate(0, [1])
    with pytest.raises(IndexError):  # free queue empty: deque[0]
        cache.allocate(1, [5, 6])
    assert cache.can_allocate(0) and not cache.can_allocate(1)
    with pytest.raises(AssertionError):
        PagedKVCache(num_blocks=0)


def test_radix_cache_constructs():
    """The reference's RadixKVCache is a stub whose constructor raises (cache/radix.py:42-43); here it is built
    (tests/test_radix_cache.py covers it)."""
    assert RadixKVCache(num_blocks=4).num_free_blocks() == 4


# ---- context builders ---------------------------------------------------------
def test_prefill_slots_closed_form_and_short_table():
    cache = PagedKVCache(num_blocks=16, block_size=4)
    ctx = build_prefill_context(cache, [0, 1], [5, 3], [(7, 2), (9,)])
    assert ctx.slot_mapping == (28, 29, 30, 31, 8, 36, 37, 38)
    assert ctx.block_tables == ((7, 2), (9,)) and ctx.seq_lens == (5, 3) and ctx.max_seq_len == 5
    assert ctx.is_prefill and ctx.block_mask is None and ctx.prefix_lens is None
    short = build_prefill_context(cache, [0], [6], [(3,)])
    assert short.slot_mapping == (12, 13, 14, 15, -1, -1)  # context.py:42
    assert build_prefill_context(cache, [], [], []).max_seq_len == 0


def test_decode_slots():
    cache = PagedKVCache(num_blocks=16, block_size=4)
    ctx = build_decode_context(cache, [0, 1, 2], [5, 4, 9], [(7, 2), (9,), (1, 2)])
    assert ctx.slot_mapping == (8, 39, -1)
    assert not ctx.is_prefill and ctx.max_seq_len == 9


def test_chunked_prefill_context_reduces_to_prefill():
    cache = PagedKVCache(num_blocks=16, block_size=4)
    tables = [(7, 2, 5), (9, 4, 6)]
    plain = build_prefill_context(cache, [0, 1], [9, 6], tables)
    chunked0 = build_chunked_prefill_context(cache, [0, 1], [0, 0], [9, 6], tables)
    assert chunked0.slot_mapping == plain.slot_mapping and chunked0.seq_lens == plain.seq_lens
    chunked = build_chunked_prefill_context(cache, [0, 1], [4, 4], [5, 2], tables)
    assert chunked.slot_mapping == plain.slot_mapping[4:9] + plain.slot_mapping[9 + 4 : 9 + 6]
    assert chunked.seq_lens == (9, 6) and chunked.prefix_lens == (4, 4) and chunked.is_prefill


def test_inference_context_is_frozen_and_positional():
    ctx = InferenceContext(True, (1,), ((0,),), (1,), 1, None)
    with pytest.raises(Exception):
        ctx.is_prefill = False
    assert InferenceContext(is_prefill=False).slot_mapping is None


def test_large_batch_tables_share_prefix_blocks():
    """32 sequences with a common 8-block prefix get identical leading block ids."""
    cache = PagedKVCache(num_blocks=256, block_size=16)
    rng = np.random.default_rng(0)
    prefix = rng.integers(0, 1000, 128).tolist()
    tables = [cache.allocate(i, prefix + rng.integers(0, 1000, 20).tolist()) for i in range(32)]
    assert all(t[:8] == tables[0][:8] for t in tables)
    own = [b for t in tables for b in t[8:]]
    assert len(set(own)) == len(own) and not set(own) & set(tables[0][:8])
    assert cache.blocks[tables[0][0]].ref_count == 32
