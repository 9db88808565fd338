"""The engine on the GPU against the checker's restatement of the reference engine's cache-less loop
(full recompute every step, engine.py:218-250) on the same random weights: greedy tokens must be identical and
log probabilities equal to tolerance, whatever the cache type, prefix sharing or preemption does underneath."""

import pytest
import torch

from oracle import model_oracle as mo
from research_amd.inference import (CacheConfig, EngineConfig, HipPagedAttentionBackend, InferenceEngine, ModelConfig,
                                    PagedLlama, SamplingParams)
from tests.gpu_helpers import announce

pytestmark = pytest.mark.gpu

CFG = ModelConfig(vocab_size=211, hidden_size=128, intermediate_size=256, num_layers=2, num_heads=4, num_kv_heads=2,
                  head_dim=32, max_position_embeddings=512)


def _engine(dtype, cache_type, num_blocks, block_size=16, seed=0, max_batch_size=8, eos=None, use_graphs=False):
    backend = HipPagedAttentionBackend(CacheConfig(
        num_layers=CFG.num_layers, num_kv_heads=CFG.num_kv_heads, head_dim=CFG.head_dim, num_blocks=num_blocks,
        block_size=block_size, device="cuda", dtype=dtype))
    torch.manual_seed(seed)
    model = PagedLlama(CFG, backend).to(dtype).cuda().eval()
    config = EngineConfig(model_path="", cache_type=cache_type, block_size=block_size, max_batch_size=max_batch_size,
                          max_model_len=512, eos_token_id=eos, use_graphs=use_graphs)
    engine = InferenceEngine(config, model=model)
    weights = {k: v.detach().float().cpu() for k, v in model.state_dict().items()}
    return engine, weights


def _prompts():
    g = torch.Generator().manual_seed(9)
    shared = torch.randint(0, 211, (37,), generator=g).tolist()
    return [shared, shared, shared, torch.randint(0, 211, (5,), generator=g).tolist(),
            torch.randint(0, 211, (64,), generator=g).tolist(), shared[:32] + [1, 2, 3]]


def _by_prompt(samples):
    out = {}
    for s in samples:
        out.setdefault(s.prompt_tokens, []).append(s)
    return out


@pytest.mark.parametrize("cache_type", ["radix", "paged", "none"])
def test_greedy_generation_equals_full_recompute(cache_type):
    announce(f"engine fp32 {cache_type}")
    engine, weights = _engine(torch.float32, cache_type, num_blocks=64)
    prompts = _prompts()
    with torch.no_grad():
        want = mo.generate_recompute(weights, CFG, prompts, max_tokens=20)
    got = _by_prompt(engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=20)))
    assert sum(len(v) for v in got.values()) == len(prompts)
    for prompt, (tokens, logprobs, reason) in zip(prompts, want):
        for sample in got[tuple(prompt)]:
            assert list(sample.completion_tokens) == tokens, (cache_type, len(prompt))
            assert sample.logprobs == pytest.approx(logprobs, abs=2e-4)
            assert sample.finish_reason == reason and sample.weight_version == 0 and sample.ref_logprobs is None
    assert not engine.has_pending() and engine.step() == []
    if cache_type != "none":
        assert engine.cache.num_free_blocks() == 64  # everything was released
    if cache_type == "radix":
        assert engine.cache.match_prefix(prompts[0]) == 32  # the prompt's full blocks are still in the tree


def test_stop_tokens_and_eos():
    announce("engine stop rules")
    engine, weights = _engine(torch.float32, "radix", num_blocks=32)
    prompt = _prompts()[3]
    with torch.no_grad():
        (tokens, _, _), = mo.generate_recompute(weights, CFG, [prompt], max_tokens=12)
    stop = tokens[4]
    cut = tokens.index(stop) + 1
    (sample,) = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, stop_token_ids=frozenset({stop})))
    assert list(sample.completion_tokens) == tokens[:cut] and sample.finish_reason == "stop"
    engine2, _ = _engine(torch.float32, "radix", num_blocks=32, eos=stop)
    (sample,) = engine2.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12))
    assert list(sample.completion_tokens) == tokens[:cut] and sample.finish_reason == "length"  # as the reference labels it


def test_preemption_is_transparent():
    """A pool too small for every sequence to finish at once: sequences are preempted, prefilled again later,
    and still produce the tokens of the full-recompute loop."""
    announce("engine preemption")
    engine, weights = _engine(torch.float32, "radix", num_blocks=11, block_size=8)
    g = torch.Generator().manual_seed(12)
    prompts = [torch.randint(0, 211, (15,), generator=g).tolist() for _ in range(4)]
    with torch.no_grad():
        want = mo.generate_recompute(weights, CFG, prompts, max_tokens=30)
    got = _by_prompt(engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=30)))
    assert engine.num_preemptions > 0
    for prompt, (tokens, logprobs, _) in zip(prompts, want):
        (sample,) = got[tuple(prompt)]
        assert list(sample.completion_tokens) == tokens
        assert sample.logprobs == pytest.approx(logprobs, abs=2e-4)
    with pytest.raises(RuntimeError, match="cannot hold"):
        engine.generate([list(range(100))], SamplingParams(temperature=0.0, max_tokens=2))
    engine.shutdown()


def test_decode_from_captured_graphs():
    """use_graphs: every decode step replays one captured forward pass (per batch-size bucket) with its integer
    inputs rewritten in place; prefills, sampling and allocator work run eagerly between the replays.  Tokens
    must equal the full-recompute loop on every step, for batches of different sizes and paddings, through
    preemption, and after a weight update (the graph reads the parameters in place)."""
    announce("engine graphs")
    engine, weights = _engine(torch.float32, "radix", num_blocks=64, use_graphs=True, max_batch_size=16)
    prompts = _prompts()
    g = torch.Generator().manual_seed(21)
    more = prompts + [torch.randint(0, 211, (n,), generator=g).tolist() for n in (3, 17, 33, 40, 9)]
    for batch, max_tokens in ((prompts, 20), (prompts[:3], 9), (more, 12)):  # buckets of 8, 8 and 16 rows
        with torch.no_grad():
            want = mo.generate_recompute(weights, CFG, batch, max_tokens=max_tokens)
        got = _by_prompt(engine.generate(batch, SamplingParams(temperature=0.0, max_tokens=max_tokens)))
        for prompt, (tokens, logprobs, _) in zip(batch, want):
            for sample in got[tuple(prompt)]:
                assert list(sample.completion_tokens) == tokens
                assert sample.logprobs == pytest.approx(logprobs, abs=2e-4)
    assert sorted(engine._decode_graphs) == [8, 16]
    # new weights are read by the same graphs
    torch.manual_seed(3)
    fresh = PagedLlama(CFG, engine.backend).float()
    state = {k: v.cuda() for k, v in fresh.state_dict().items()}
    engine.update_weights(state)
    engine.flush_cache()
    new_weights = {k: v.float().cpu() for k, v in state.items()}
    with torch.no_grad():
        want = mo.generate_recompute(new_weights, CFG, prompts[:4], max_tokens=10)
    got = _by_prompt(engine.generate(prompts[:4], SamplingParams(temperature=0.0, max_tokens=10)))
    for prompt, (tokens, _, _) in zip(prompts[:4], want):
        for sample in got[tuple(prompt)]:
            assert list(sample.completion_tokens) == tokens
    # a pool too small for all sequences at once: preemption between replays
    engine2, weights2 = _engine(torch.float32, "radix", num_blocks=11, block_size=8, use_graphs=True)
    g = torch.Generator().manual_seed(12)
    small = [torch.randint(0, 211, (15,), generator=g).tolist() for _ in range(4)]
    with torch.no_grad():
        want = mo.generate_recompute(weights2, CFG, small, max_tokens=30)
    got = _by_prompt(engine2.generate(small, SamplingParams(temperature=0.0, max_tokens=30)))
    assert engine2.num_preemptions > 0
    for prompt, (tokens, _, _) in zip(small, want):
        (sample,) = got[tuple(prompt)]
        assert list(sample.completion_tokens) == tokens


def test_rollouts_of_one_prompt_prefill_in_two_passes():
    """Rows with no cached prefix and rows with one are prefilled in separate passes when that removes most of
    the padding (N rollouts of a prompt = one full row + N-1 one-token rows); results are those of the
    full-recompute loop either way."""
    announce("engine two-pass prefill")
    engine, weights = _engine(torch.float32, "radix", num_blocks=64)
    g = torch.Generator().manual_seed(31)
    a = torch.randint(0, 211, (64,), generator=g).tolist()
    b = torch.randint(0, 211, (48,), generator=g).tolist()
    prompts = [a, a, a, a, b, b, b]
    calls = []
    rows = engine._prefill_rows
    engine._prefill_rows = lambda seqs, cached, chunks: (calls.append((len(seqs), max(chunks))), rows(seqs, cached, chunks))[1]
    with torch.no_grad():
        want = mo.generate_recompute(weights, CFG, [a, b], max_tokens=10)
    got = _by_prompt(engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10)))
    assert calls == [(2, 64), (5, 1)]  # the two first occurrences, then the five rollouts that found their prompt cached
    for prompt, (tokens, logprobs, _) in zip([a, b], want):
        assert len(got[tuple(prompt)]) == (4 if prompt is a else 3)
        for sample in got[tuple(prompt)]:
            assert list(sample.completion_tokens) == tokens
            assert sample.logprobs == pytest.approx(logprobs, abs=2e-4)


def _fp8_engine(use_graphs):
    backend = HipPagedAttentionBackend(CacheConfig(
        num_layers=CFG.num_layers, num_kv_heads=CFG.num_kv_heads, head_dim=CFG.head_dim, num_blocks=64,
        block_size=16, device="cuda", dtype=torch.bfloat16, kv_format="fp8_e4m3"))
    torch.manual_seed(1)
    model = PagedLlama(CFG, backend).to(torch.bfloat16).cuda().eval()
    engine = InferenceEngine(EngineConfig(model_path="", cache_type="radix", max_batch_size=8, max_model_len=512,
                                          use_graphs=use_graphs), model=model)
    return engine, {k: v.detach().float().cpu() for k, v in model.state_dict().items()}


def test_decode_graphs_on_an_fp8_pool():
    """use_graphs with an fp8-e4m3 pool: the append's block list is computed on the device inside the captured
    pass.  A full bucket (8 unrelated prompts, all finishing together) replays exactly the launches of the eager
    engine, so tokens and log probabilities are those of the eager engine; a padded bucket (6 prompts, some
    sharing a prefix) is held to the full-precision checker like the eager fp8 engine."""
    announce("engine fp8 pool with graphs")
    g = torch.Generator().manual_seed(44)
    full = [torch.randint(0, 211, (n,), generator=g).tolist() for n in (5, 16, 17, 31, 40, 9, 23, 12)]
    eager, _ = _fp8_engine(False)
    want = _by_prompt(eager.generate(full, SamplingParams(temperature=0.0, max_tokens=14)))
    engine, weights = _fp8_engine(True)
    got = _by_prompt(engine.generate(full, SamplingParams(temperature=0.0, max_tokens=14)))
    assert sorted(engine._decode_graphs) == [8]
    for prompt in full:
        (a,), (b,) = got[tuple(prompt)], want[tuple(prompt)]
        assert a.completion_tokens == b.completion_tokens
        assert a.logprobs == pytest.approx(b.logprobs, abs=1e-6)
    assert torch.equal(engine.backend.k_cache.view(torch.uint8), eager.backend.k_cache.view(torch.uint8))
    assert torch.equal(engine.backend.v_scale, eager.backend.v_scale)
    samples = engine.generate(_prompts(), SamplingParams(temperature=0.0, max_tokens=12))
    assert len(samples) == 6
    for s in samples:
        with torch.no_grad():
            ref = mo.logprobs_of(weights, CFG, list(s.prompt_tokens + s.completion_tokens), len(s.prompt_tokens))
        assert s.logprobs == pytest.approx(ref, abs=0.25)


def test_max_model_len_beyond_the_rotary_table_is_refused():
    backend = HipPagedAttentionBackend(CacheConfig(
        num_layers=CFG.num_layers, num_kv_heads=CFG.num_kv_heads, head_dim=CFG.head_dim, num_blocks=16,
        block_size=16, device="cuda", dtype=torch.bfloat16))
    model = PagedLlama(CFG, backend).to(torch.bfloat16).cuda().eval()
    with pytest.raises(ValueError, match="max_position_embeddings"):
        InferenceEngine(EngineConfig(model_path="", cache_type="radix", max_model_len=CFG.max_position_embeddings + 1),
                        model=model)


def test_bf16_generation_and_weight_update():
    announce("engine bf16, update_weights, flush_cache")
    engine, weights = _engine(torch.bfloat16, "radix", num_blocks=64, seed=1)
    prompts = _prompts()
    samples = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16), num_samples_per_prompt=2)
    assert len(samples) == 2 * len(prompts)
    for s in samples:  # teacher-forced log probabilities of the engine's own tokens under the checker
        with torch.no_grad():
            want = mo.logprobs_of(weights, CFG, list(s.prompt_tokens + s.completion_tokens), len(s.prompt_tokens))
        assert s.logprobs == pytest.approx(want, abs=0.08)
    # sampling at temperature 1: log probabilities still describe the unscaled distribution
    torch.manual_seed(5)
    hot = engine.generate(prompts[:2], SamplingParams(temperature=1.0, max_tokens=8))
    for s in hot:
        with torch.no_grad():
            want = mo.logprobs_of(weights, CFG, list(s.prompt_tokens + s.completion_tokens), len(s.prompt_tokens))
        assert s.logprobs == pytest.approx(want, abs=0.08)
    # new weights: version counts up, the cache is flushed, results follow the new weights
    torch.manual_seed(2)
    fresh = PagedLlama(CFG, engine.backend).to(torch.bfloat16)
    state = {k: v.cuda() for k, v in fresh.state_dict().items()}
    engine.update_weights(state)
    assert engine.get_weight_version() == 1
    assert engine.cache.match_prefix(prompts[0]) == 32
    engine.flush_cache()
    assert engine.cache.match_prefix(prompts[0]) == 0 and not engine.backend.k_cache.any()
    new_weights = {k: v.float().cpu() for k, v in state.items()}
    (s,) = engine.generate(prompts[:1], SamplingParams(temperature=0.0, max_tokens=8))
    assert s.weight_version == 1
    with torch.no_grad():
        want = mo.logprobs_of(new_weights, CFG, list(s.prompt_tokens + s.completion_tokens), len(s.prompt_tokens))
    assert s.logprobs == pytest.approx(want, abs=0.08)


def test_engine_on_an_fp8_pool():
    """The same model with an fp8-e4m3 KV pool: rotary append into fp8 blocks, chunked prefill over dequantised
    blocks, fp8 decode.  Teacher-forced log probabilities stay close to the full-precision checker."""
    announce("engine fp8 pool")
    backend = HipPagedAttentionBackend(CacheConfig(
        num_layers=CFG.num_layers, num_kv_heads=CFG.num_kv_heads, head_dim=CFG.head_dim, num_blocks=64,
        block_size=16, device="cuda", dtype=torch.bfloat16, kv_format="fp8_e4m3"))
    torch.manual_seed(1)
    model = PagedLlama(CFG, backend).to(torch.bfloat16).cuda().eval()
    engine = InferenceEngine(EngineConfig(model_path="", cache_type="radix", max_batch_size=8, max_model_len=512),
                             model=model)
    weights = {k: v.detach().float().cpu() for k, v in model.state_dict().items()}
    samples = engine.generate(_prompts(), SamplingParams(temperature=0.0, max_tokens=12))
    assert len(samples) == 6
    for s in samples:
        with torch.no_grad():
            want = mo.logprobs_of(weights, CFG, list(s.prompt_tokens + s.completion_tokens), len(s.prompt_tokens))
        assert s.logprobs == pytest.approx(want, abs=0.25)
