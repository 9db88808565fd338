"""Scheduling, block accounting and preemption of the engine on the host: the queues, the scheduler and the
allocators run as they are, the model's forward passes are replaced by a stand-in that appends a fixed token
(no GPU, no kernels)."""

import random
from types import SimpleNamespace

import pytest

from research_amd.inference.cache import CountingPagedKVCache, RadixKVCache
from research_amd.inference.engine import InferenceEngine
from research_amd.inference.types import EngineConfig, SamplingParams, SchedulerConfig


class HostEngine(InferenceEngine):
    """The engine with `_prefill_rows` / `_decode_rows` (the two places that run the model) stubbed."""

    def __init__(self, num_blocks, block_size, cache_type, max_batch_size=8, max_model_len=4096):
        self.config = EngineConfig(model_path="", cache_type=cache_type, block_size=block_size,
                                   max_batch_size=max_batch_size, max_model_len=max_model_len,
                                   num_kv_blocks=num_blocks)
        self.backend = SimpleNamespace(config=SimpleNamespace(num_blocks=num_blocks, block_size=block_size),
                                       clear_cache=lambda: None)
        self.tokenizer = None
        self.scheduler_config = SchedulerConfig(max_batch_size=max_batch_size,
                                                max_tokens_per_batch=max_batch_size * 512, block_size=block_size)
        self.cache = self._new_cache()
        self.waiting, self.running = [], []
        self.seq_counter = self.weight_version = self.num_preemptions = 0
        self._decode_graphs = {}
        self.max_blocks_in_use = 0

    def _emit(self, seqs):
        bs = self.config.block_size
        for s in seqs:  # every sequence that computes holds blocks for all its tokens
            assert len(s.block_ids) * bs >= len(s.token_ids), (s.seq_id, len(s.block_ids), len(s.token_ids))
        self.max_blocks_in_use = max(self.max_blocks_in_use,
                                     self.backend.config.num_blocks - self.cache.num_free_blocks())
        finished = []
        for s in seqs:
            s.append_token(7, -0.5)
            if self._should_stop(s, 7):
                from research_amd.inference.types import SequenceStatus
                s.status = SequenceStatus.FINISHED
                self.cache.deallocate(s.seq_id)
                finished.append(s)
        return finished

    def _prefill_rows(self, seqs, cached, chunks):
        return self._emit(seqs)

    def _decode_rows(self, seqs):
        return self._emit(seqs)


def _owned_blocks(cache):
    if isinstance(cache, CountingPagedKVCache):
        return {b for blocks in cache.seq_to_blocks.values() for b in blocks}
    return None


@pytest.mark.parametrize("cache_type", ["paged", "radix"])
def test_prefill_admitted_in_the_step_whose_decodes_take_the_last_block(cache_type):
    """Block size 4, pool of 4.  A holds one block and its next decode starts a second one; B's prompt needs
    all three blocks that are free before that decode.  B must wait, nothing may raise, no block may be lost."""
    e = HostEngine(num_blocks=4, block_size=4, cache_type=cache_type)
    a = e.add_request([1, 2, 3, 4], SamplingParams(max_tokens=6))
    assert e.step() == []                     # A prefilled: 4 tokens + 1 sampled = 5, one block held
    assert len(e.running) == 1 and e.cache.num_free_blocks() == 3
    e.add_request(list(range(10, 22)), SamplingParams(max_tokens=2))  # B: 12 tokens = 3 blocks = all free ones
    # this step: A's decode writes position 4 = first token of a new block, leaving 2 free; B needs 3
    e.step()
    assert [s.seq_id for s in e.running] == [a] and len(e.waiting) == 1
    assert e.waiting[0].block_ids == []
    results = []
    while e.has_pending():
        results += e.step()
    assert len(results) == 2
    assert e.cache.num_free_blocks() == 4
    owned = _owned_blocks(e.cache)
    assert owned is None or owned == set()


@pytest.mark.parametrize("cache_type", ["paged", "radix"])
def test_counting_allocator_refuses_without_a_trace(cache_type):
    cls = CountingPagedKVCache if cache_type == "paged" else RadixKVCache
    c = cls(4, 4)
    c.allocate(0, list(range(9)))             # 3 blocks
    with pytest.raises(RuntimeError, match="No free blocks"):
        c.allocate(1, list(range(100, 108)))  # 2 blocks, 1 free
    assert c.num_free_blocks() == 1 and c.get_block_ids(1) == ()
    c.allocate(2, [5, 6, 7])                  # the free block is still usable
    assert c.num_free_blocks() == 0
    c.deallocate(0)
    c.deallocate(2)
    assert c.num_free_blocks() == 4


def test_blocks_needed_counts_shared_prefix_blocks_only_while_held():
    c = CountingPagedKVCache(8, 4)
    prompt = list(range(12))
    c.allocate(0, prompt + [99])               # 3 full blocks + 1 partial
    assert c.blocks_needed(prompt + [50, 51]) == 1   # the three full blocks are shared, the tail is new
    c.deallocate(0)
    assert c.blocks_needed(prompt + [50, 51]) == 4   # cached blocks nobody holds come out of the free queue
    got = c.allocate(1, prompt + [50, 51])
    assert len(got) == 4 and c.num_free_blocks() == 4


@pytest.mark.parametrize("cache_type", ["paged", "radix"])
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_tight_pool_random_traffic_never_raises_and_returns_every_block(cache_type, seed):
    """Many requests against a pool that holds only a few of them at a time, with shared prompts, so that
    preemption, deferred prefills and prefix reuse all happen; every request finishes with its full length."""
    rng = random.Random(seed)
    bs, blocks = 4, 24
    e = HostEngine(num_blocks=blocks, block_size=bs, cache_type=cache_type, max_batch_size=6)
    prompts = [[rng.randrange(100) for _ in range(rng.randrange(1, 30))] for _ in range(5)]
    want = {}
    pending = 0
    for step in range(400):
        if pending < 40 and rng.random() < 0.5:
            p = list(rng.choice(prompts)) if rng.random() < 0.6 else [rng.randrange(100) for _ in range(rng.randrange(1, 40))]
            n = rng.randrange(1, 25)
            want[e.add_request(p, SamplingParams(max_tokens=n))] = (len(p), n)
            pending += 1
        for sample in e.step():
            pending -= 1
            assert len(sample.completion_tokens) >= 1
        used = blocks - e.cache.num_free_blocks()
        held = sum(len(s.block_ids) for s in e.running)
        assert used <= held            # shared blocks are counted once, nothing is held by nobody
    while e.has_pending():
        for sample in e.step():
            pending -= 1
    assert pending == 0
    assert e.cache.num_free_blocks() == blocks
    assert e.max_blocks_in_use <= blocks
