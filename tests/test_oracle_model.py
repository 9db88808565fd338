"""Pins the checker's model forward against HuggingFace's Llama implementation (the class the reference's
engine instantiates through AutoModelForCausalLM, engine.py:60-68) on random weights, and checks the
scheduler / sampling mirrors against the facts their reference statements fix."""

import pytest
import torch

from oracle import model_oracle as mo
from research_amd.inference.model import ModelConfig
from research_amd.inference.sampling import compute_logprobs_for_tokens, sample_greedy, sample_with_logprobs
from research_amd.inference.scheduler import can_schedule_any, schedule
from research_amd.inference.types import SchedulerConfig, Sequence, SequenceStatus


def _hf(num_kv_heads):
    from transformers import LlamaConfig, LlamaForCausalLM

    hf_cfg = LlamaConfig(vocab_size=97, hidden_size=64, intermediate_size=112, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=num_kv_heads, head_dim=16,
                         max_position_embeddings=256, rope_theta=10000.0, rms_norm_eps=1e-5,
                         tie_word_embeddings=False, attention_bias=False)
    torch.manual_seed(0)
    model = LlamaForCausalLM(hf_cfg).eval()
    return model, ModelConfig.from_hf_dict(hf_cfg.to_dict())


@pytest.mark.parametrize("num_kv_heads", [4, 2, 1])
def test_forward_equals_huggingface_llama(num_kv_heads):
    model, cfg = _hf(num_kv_heads)
    assert (cfg.num_layers, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim) == (2, 4, num_kv_heads, 16)
    ids = torch.randint(0, 97, (3, 19), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        want = model(ids).logits
        got = mo.llama_forward(dict(model.state_dict()), cfg, ids)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
    # causal: changing later tokens leaves earlier logits alone
    ids2 = ids.clone()
    ids2[:, 10:] = (ids2[:, 10:] + 1) % 97
    with torch.no_grad():
        got2 = mo.llama_forward(dict(model.state_dict()), cfg, ids2)
    torch.testing.assert_close(got2[:, :10], got[:, :10], rtol=0, atol=1e-6)
    assert not torch.allclose(got2[:, 10:], got[:, 10:])


def test_generation_loop_rules():
    model, cfg = _hf(2)
    w = dict(model.state_dict())
    with torch.no_grad():
        (toks, lps, reason), = mo.generate_recompute(w, cfg, [[5, 6, 7]], max_tokens=4)
        assert len(toks) == 4 and len(lps) == 4 and reason == "length"
        first = int(mo.llama_forward(w, cfg, torch.tensor([[5, 6, 7]]))[0, -1].argmax())
        assert toks[0] == first and all(lp <= 0 for lp in lps)
        (toks2, _, reason2), = mo.generate_recompute(w, cfg, [[5, 6, 7]], max_tokens=4,
                                                     stop_token_ids=frozenset({toks[1]}))
        assert toks2 == toks[:2] and reason2 == "stop"
        assert mo.logprobs_of(w, cfg, [5, 6, 7] + toks, 3) == pytest.approx(lps, abs=1e-5)


# ---- scheduler (scheduler.py:15-108) -------------------------------------------------------------------------
def _seq(i, n, status):
    return Sequence(seq_id=i, token_ids=list(range(n)), block_ids=[], num_prompt_tokens=n, status=status,
                    temperature=1.0, max_tokens=8, stop_token_ids=frozenset(), output_logprobs=[])


def test_schedule_limits():
    W, R = SequenceStatus.WAITING, SequenceStatus.RUNNING
    cfg = SchedulerConfig(max_batch_size=4, max_tokens_per_batch=40, block_size=4)
    running = [_seq(0, 5, R), _seq(1, 9, R)]
    waiting = [_seq(2, 10, W), _seq(3, 10, W), _seq(4, 30, W), _seq(5, 1, W)]
    out = schedule(waiting, running, num_free_blocks=100, config=cfg)
    assert out.decode_seqs == (0, 1) and out.prefill_seqs == (2, 3) and out.preempted_seqs == ()  # batch of 4 is full
    cfg8 = SchedulerConfig(max_batch_size=8, max_tokens_per_batch=40, block_size=4)
    out = schedule(waiting, running, 100, cfg8)
    assert out.prefill_seqs == (2, 3)  # 2 + 10 + 10 + 30 > 40: admission stops, sequence 5 is not tried
    out = schedule(waiting, running, num_free_blocks=5, config=cfg8)
    assert out.prefill_seqs == (2,)  # 3 blocks, then 3 more do not fit into the 2 left
    out = schedule(waiting, running, num_free_blocks=2, config=cfg8)
    assert out.prefill_seqs == () and out.decode_seqs == (0, 1)
    one = SchedulerConfig(max_batch_size=1, max_tokens_per_batch=40, block_size=4)
    out = schedule([], running, 100, one)
    assert out.decode_seqs == (0,) and out.preempted_seqs == (1,)
    with pytest.raises(AssertionError):
        schedule(running, [], 100, cfg)  # a RUNNING sequence in the waiting queue
    assert can_schedule_any([], running, 0, cfg) and not can_schedule_any([], [], 10, cfg)
    assert can_schedule_any(waiting, [], 3, cfg) and not can_schedule_any(waiting, [], 2, cfg)


# ---- sampling (sampling.py:11-103) -----------------------------------------------------------------------------
def test_sampling_facts():
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(5, 11, generator=g)
    temps = torch.tensor([0.0, 1.0, 0.0, 0.5, 2.0])
    torch.manual_seed(7)
    tokens, lps = sample_with_logprobs(logits, temps)
    assert tokens[0] == logits[0].argmax() and tokens[2] == logits[2].argmax()
    ref = torch.log_softmax(logits, -1)  # always the unscaled distribution
    torch.testing.assert_close(lps, ref[torch.arange(5), tokens])
    gt, gl = sample_greedy(logits)
    assert torch.equal(gt, logits.argmax(-1)) and torch.equal(gl, ref.max(-1).values)
    # the empirical distribution follows softmax(logits / T)
    row = torch.tensor([[2.0, 1.0, 0.0, -1.0]]).repeat(20000, 1)
    torch.manual_seed(11)
    drawn, _ = sample_with_logprobs(row, torch.full((20000,), 0.5))
    freq = torch.bincount(drawn, minlength=4).float() / 20000
    torch.testing.assert_close(freq, torch.softmax(row[0] / 0.5, -1), atol=0.01, rtol=0)
    lp = compute_logprobs_for_tokens(logits[None], tokens[None])
    torch.testing.assert_close(lp[0], lps)
    with pytest.raises(AssertionError):
        sample_with_logprobs(logits, temps[:3])
