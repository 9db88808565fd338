"""Scheduling as a pure function (reference: rollouts/rollouts/inference/scheduler.py:15-108).

Running sequences decode first (one token each); waiting sequences are then
admitted for prefill, in order, until the batch size, the token budget or the
free KV blocks run out.  Nothing is mutated.
"""

from __future__ import annotations

from typing import List

from .types import SchedulerConfig, SchedulerOutput, Sequence, SequenceStatus


def _blocks_for(num_tokens: int, block_size: int) -> int:
    return (num_tokens + block_size - 1) // block_size


def schedule(waiting: List[Sequence], running: List[Sequence], num_free_blocks: int,
             config: SchedulerConfig) -> SchedulerOutput:
    """What to run this step (scheduler.py:15-83).

    Every running sequence decodes unless the batch is already full, in which case it is reported as preempted.
    Waiting sequences are admitted first-come-first-served and admission stops at the first one that does not
    fit (batch slots, ``max_tokens_per_batch`` counting one token per decode and the whole prompt per prefill,
    or blocks for the whole prompt).
    """
    assert config.max_batch_size > 0
    assert config.block_size > 0
    decode, preempted = [], []
    for seq in running:
        assert seq.status == SequenceStatus.RUNNING, f"Expected RUNNING, got {seq.status}"
        (decode if len(decode) < config.max_batch_size else preempted).append(seq.seq_id)
    tokens = len(decode)
    blocks = num_free_blocks
    prefill = []
    for seq in waiting:
        assert seq.status == SequenceStatus.WAITING, f"Expected WAITING, got {seq.status}"
        n = len(seq.token_ids)
        need = _blocks_for(n, config.block_size)
        if (len(prefill) + len(decode) >= config.max_batch_size or tokens + n > config.max_tokens_per_batch
                or need > blocks):
            break
        prefill.append(seq.seq_id)
        blocks -= need
        tokens += n
    return SchedulerOutput(prefill_seqs=tuple(prefill), decode_seqs=tuple(decode), preempted_seqs=tuple(preempted))


def can_schedule_any(waiting: List[Sequence], running: List[Sequence], num_free_blocks: int,
                     config: SchedulerConfig) -> bool:
    """True when a step would do work: something is running, or the first waiting prompt fits the free blocks
    (scheduler.py:86-108)."""
    if running:
        return True
    if not waiting:
        return False
    return _blocks_for(len(waiting[0].token_ids), config.block_size) <= num_free_blocks
