"""Prefix-tree allocator (the reference declares it as a stub, cache/radix.py:26-61, behind the protocol of
cache/protocol.py:9-43).  There is no reference behaviour to match beyond the protocol, so the tests pin the
protocol's contracts, the sharing the stub's docstring promises (N rollouts of one prompt share their prefix
blocks), and the allocator's invariants under random operation sequences against a brute-force model."""

import random

import pytest

from research_amd.inference import allocate_and_build_context, extend_and_build_context
from research_amd.inference.cache import KVCacheManager, PagedKVCache, RadixKVCache


def test_protocol_surface():
    cache = RadixKVCache(num_blocks=8, block_size=4)
    for name in ("num_free_blocks", "can_allocate", "allocate", "deallocate", "append_token", "get_block_ids"):
        assert callable(getattr(cache, name)) and hasattr(KVCacheManager, name)
    assert cache.block_size == 4 and cache.num_free_blocks() == 8
    assert cache.can_allocate(32) and not cache.can_allocate(33)
    assert cache.get_block_ids(5) == () and cache.get_cached_tokens(5) == 0
    cache.deallocate(5)  # unknown sequence: nothing happens, as in PagedKVCache
    with pytest.raises(AssertionError):
        RadixKVCache(num_blocks=0)


def test_same_facts_as_the_paged_allocator_on_the_reference_scenario():
    """The integer facts the reference's test asserts for PagedKVCache (examples/inference/test_kv_cache.py:117-178:
    20 tokens -> 2 blocks, 14 free, 16 free after deallocate; a second sequence with the same 8 leading tokens
    has 8 cached) hold for the tree as well."""
    for cls in (PagedKVCache, RadixKVCache):
        cache = cls(num_blocks=16, block_size=16)
        blocks = cache.allocate(0, list(range(20)))
        assert len(blocks) == 2 and cache.num_free_blocks() == 14
        cache.deallocate(0)
        assert cache.num_free_blocks() == 16
        cache = cls(num_blocks=16, block_size=4)
        a = cache.allocate(0, [1, 2, 3, 4, 5, 6, 7, 8, 9])
        b = cache.allocate(1, [1, 2, 3, 4, 5, 6, 7, 8, 10, 11])
        assert a[:2] == b[:2] and a[2] != b[2]
        assert cache.get_cached_tokens(0) == 0 and cache.get_cached_tokens(1) == 8


def test_rollouts_of_one_prompt_share_the_prefix():
    cache = RadixKVCache(num_blocks=32, block_size=4)
    prompt = list(range(100, 110))  # 2 full blocks + 2 tokens
    tables = [cache.allocate(i, prompt) for i in range(8)]
    shared = tables[0][:2]
    assert all(t[:2] == shared for t in tables)
    assert len({t[2] for t in tables}) == 8  # every rollout has its own partial block
    assert cache.num_free_blocks() == 32 - 2 - 8
    assert [cache.get_cached_tokens(i) for i in range(8)] == [0] + [8] * 7
    # rollouts diverge: each fills its third block with its own tokens, then starts a fourth
    for i in range(8):
        assert cache.append_token(i, 1000 + i) is None
        assert cache.append_token(i, 2000 + i) is None  # block 3 full now: it joins the tree
        fresh = cache.append_token(i, 3000 + i)
        assert fresh is not None and cache.get_block_ids(i)[-1] == fresh and len(cache.get_block_ids(i)) == 4
    # a new sequence that repeats rollout 3 up to its third block hits all three
    cache.allocate(99, prompt + [1003, 2003, 7])
    assert cache.get_cached_tokens(99) == 12 and cache.get_block_ids(99)[:3] == cache.get_block_ids(3)[:3]
    for i in list(range(8)) + [99]:
        cache.deallocate(i)
    assert cache.num_free_blocks() == 32
    # everything stays cached until the space is needed
    assert cache.match_prefix(prompt + [1003, 2003]) == 12


def test_two_sequences_filling_equal_blocks_keep_private_copies():
    cache = RadixKVCache(num_blocks=8, block_size=2)
    cache.allocate(0, [1])
    cache.allocate(1, [1])
    assert cache.append_token(0, 2) is None  # joins the tree
    assert cache.append_token(1, 2) is None  # an equal node exists: stays private
    assert cache.get_block_ids(0) != cache.get_block_ids(1)
    assert cache.append_token(1, 3) is not None and len(cache.get_block_ids(1)) == 2
    cache.allocate(2, [1, 2, 9])
    assert cache.get_block_ids(2)[0] == cache.get_block_ids(0)[0] and cache.get_cached_tokens(2) == 2


def test_eviction_is_lru_and_leaves_first_and_never_touches_live_blocks():
    cache = RadixKVCache(num_blocks=6, block_size=2)
    cache.allocate(0, [1, 2, 3, 4])      # nodes A(1,2) -> B(3,4)
    cache.allocate(1, [5, 6])            # node C(5,6)
    cache.allocate(2, [1, 2, 7, 8, 9])   # shares A, node D(7,8), private block
    live2 = cache.get_block_ids(2)
    assert cache.num_free_blocks() == 1
    cache.deallocate(0)                   # B idle (A still held by sequence 2)
    cache.deallocate(1)                   # C idle, more recent than B
    assert cache.num_free_blocks() == 3 and cache.match_prefix([1, 2, 3, 4]) == 4 and cache.match_prefix([5, 6]) == 2
    cache.allocate(3, [20, 21, 22, 23])   # takes the free block, then evicts B (least recently used)
    assert cache.match_prefix([1, 2, 3, 4]) == 2 and cache.match_prefix([5, 6]) == 2
    assert cache.get_block_ids(2) == live2
    assert set(cache.get_block_ids(3)).isdisjoint(live2)
    cache.allocate(4, [30, 31])           # evicts C
    assert cache.match_prefix([5, 6]) == 0 and cache.num_free_blocks() == 0
    assert not cache.can_allocate(1)
    with pytest.raises(RuntimeError, match="No free blocks"):
        cache.allocate(5, [40])
    with pytest.raises(RuntimeError, match="No free blocks"):
        cache.append_token(4, 32)
    assert cache.get_block_ids(5) == () and cache.get_block_ids(2) == live2  # failed calls changed nothing
    # a hit revives an idle node instead of evicting it
    cache.deallocate(3)
    with pytest.raises(RuntimeError, match="need 1 beyond the cached prefix, have 0"):
        cache.allocate(6, [20, 21, 22, 23, 24])  # the two idle blocks are its own prefix, the third is missing
    assert cache.num_free_blocks() == 2
    cache.deallocate(4)
    cache.allocate(6, [20, 21, 22, 23, 24])
    assert cache.get_cached_tokens(6) == 4 and cache.match_prefix([30, 31]) == 0


def test_context_builders_accept_the_tree():
    cache = RadixKVCache(num_blocks=8, block_size=4)
    ctx, cached = allocate_and_build_context(cache, seq_id=0, token_ids=list(range(6)))
    blocks = cache.get_block_ids(0)
    assert cached == 0 and ctx.is_prefill and ctx.seq_lens == (6,)
    assert ctx.slot_mapping == tuple(blocks[p // 4] * 4 + p % 4 for p in range(6))
    ctx = extend_and_build_context(cache, seq_id=0, new_token=6, current_len=6)
    assert ctx.seq_lens == (7,) and ctx.slot_mapping == (blocks[1] * 4 + 2,)
    ctx = extend_and_build_context(cache, seq_id=0, new_token=7, current_len=7)
    ctx = extend_and_build_context(cache, seq_id=0, new_token=8, current_len=8)  # starts block 3
    assert len(cache.get_block_ids(0)) == 3 and ctx.slot_mapping == (cache.get_block_ids(0)[2] * 4,)


def test_random_operations_keep_the_invariants():
    rng = random.Random(5)
    bs, nb = 3, 24
    cache = RadixKVCache(num_blocks=nb, block_size=bs)
    tokens = {}  # live sequence -> its tokens
    next_id = 0
    for step in range(3000):
        op = rng.random()
        if op < 0.35:
            n = rng.randint(0, 10)
            toks = [rng.randint(0, 2) for _ in range(n)]  # tiny alphabet: many shared prefixes
            if cache.can_allocate(n):
                cached_before = cache.match_prefix(toks)
                blocks = cache.allocate(next_id, toks)
                assert len(blocks) == -(-n // bs)
                assert cache.get_cached_tokens(next_id) == cached_before
                tokens[next_id] = toks
                next_id += 1
        elif op < 0.75 and tokens:
            sid = rng.choice(list(tokens))
            before = cache.get_block_ids(sid)
            try:
                fresh = cache.append_token(sid, rng.randint(0, 2))
            except RuntimeError:
                assert cache.num_free_blocks() == 0 and len(tokens[sid]) % bs == 0
                continue
            tokens[sid].append(None)  # placeholder: only the count matters below
            after = cache.get_block_ids(sid)
            assert (fresh is not None) == (len(tokens[sid]) % bs == 1 or bs == 1)
            assert after[: len(before)] == before and len(after) == -(-len(tokens[sid]) // bs)
        elif tokens:
            sid = rng.choice(list(tokens))
            cache.deallocate(sid)
            del tokens[sid]
            assert cache.get_block_ids(sid) == ()
        # invariants
        owners = {}
        for sid in tokens:
            for pos, b in enumerate(cache.get_block_ids(sid)):
                assert 0 <= b < nb
                owners.setdefault(b, set()).add((sid, pos))
        live = set(owners)
        assert len(live) + cache.num_free_blocks() == nb, step
        for b, who in owners.items():
            assert len({pos for _, pos in who}) == 1  # a shared block sits at the same depth for every sharer
        for sid in tokens:
            assert len(set(cache.get_block_ids(sid))) == len(cache.get_block_ids(sid))
    for sid in list(tokens):
        cache.deallocate(sid)
    assert cache.num_free_blocks() == nb
