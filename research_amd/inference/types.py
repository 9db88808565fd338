"""Dataclasses of the inference package (reference: rollouts/rollouts/inference/types.py).

``InferenceContext`` (types.py:72-107) is the per-step descriptor handed to
every attention layer; its field names, order and defaults are the
reference's, so code which builds a context for the reference backend builds
one for this backend unchanged.  The engine-side types (types.py:14-69,
:110-171) keep their names, fields and defaults as well; ``EngineConfig``
gains optional fields for what the reference's engine does not have yet: a KV
pool size and an end-of-sequence token for engines built without a tokenizer.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum, auto
from typing import FrozenSet, List, Optional, Tuple


@dataclass(frozen=True)
class InferenceContext:
    """Immutable description of one forward pass over a batch.

    ``slot_mapping``  flat, one entry per input token (``batch * seq_len``);
                      the cache slot that token's K/V row is written to,
                      ``-1`` = drop the row.  ``None`` = do not touch the cache.
    ``block_tables``  ragged: for each sequence the pool block ids that hold
                      its tokens, in order.
    ``seq_lens``      decode: context length of each sequence *including* the
                      token appended in this step.
    ``block_mask``    ``None`` (the configured mask) or a ``PagedMask`` of attention/mask.py that replaces it.

    Extension (not in the reference, keyword-only in spirit, defaulted so the
    reference's positional construction still works):
    ``prefix_lens``   chunked prefill: number of tokens of each sequence that
                      are already in the cache.  When set on a prefill context
                      the chunk's queries attend over cache[0:prefix] followed
                      by the chunk itself (bottom-right aligned causal mask).
    """

    is_prefill: bool
    slot_mapping: Optional[Tuple[int, ...]] = None
    block_tables: Optional[Tuple[Tuple[int, ...], ...]] = None
    seq_lens: Optional[Tuple[int, ...]] = None
    max_seq_len: int = 0
    block_mask: Optional[object] = None
    prefix_lens: Optional[Tuple[int, ...]] = None


# --------------------------------------------------------------------------- engine configuration (types.py:14-49)


@dataclass(frozen=True)
class EngineConfig:
    """Engine configuration (types.py:14-24).  ``model_path`` names a local directory with ``config.json`` and
    safetensors weights, or is ignored when the engine is handed a model object.  Added, optional:
    ``num_kv_blocks`` (pool size; default: enough for ``max_batch_size`` sequences of ``max_model_len`` tokens,
    capped at 65 536 blocks), ``eos_token_id`` (used when there is no tokenizer), ``use_graphs`` (replay the
    decode step's forward pass from a captured HIP graph per batch-size bucket instead of launching it kernel by
    kernel)."""

    model_path: str
    cache_type: str = "none"  # "paged" | "radix" | "none"
    block_size: int = 16
    max_batch_size: int = 256
    max_model_len: int = 8192
    gpu_memory_utilization: float = 0.9
    tensor_parallel_size: int = 1
    num_kv_blocks: Optional[int] = None
    eos_token_id: Optional[int] = None
    use_graphs: bool = False


@dataclass(frozen=True)
class SamplingParams:
    """Sampling configuration (types.py:27-33)."""

    temperature: float = 1.0
    max_tokens: int = 256
    stop_token_ids: FrozenSet[int] = frozenset()


@dataclass(frozen=True)
class SchedulerConfig:
    """Scheduler limits (types.py:36-42)."""

    max_batch_size: int
    max_tokens_per_batch: int
    block_size: int


# --------------------------------------------------------------------------- outputs (types.py:50-69)


@dataclass(frozen=True)
class TrainingSample:
    """One finished sequence for RL training (types.py:50-60)."""

    prompt_tokens: Tuple[int, ...]
    completion_tokens: Tuple[int, ...]
    logprobs: Tuple[float, ...]
    ref_logprobs: Optional[Tuple[float, ...]]
    weight_version: int
    finish_reason: str  # "stop" | "length"


@dataclass(frozen=True)
class SchedulerOutput:
    """Sequence ids to prefill, decode and preempt in one step (types.py:63-69)."""

    prefill_seqs: Tuple[int, ...]
    decode_seqs: Tuple[int, ...]
    preempted_seqs: Tuple[int, ...]


# --------------------------------------------------------------------------- per-sequence state (types.py:115-171)


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


@dataclass
class Sequence:
    """Mutable state of one request while it generates (types.py:121-171)."""

    seq_id: int
    token_ids: List[int]
    block_ids: List[int]
    num_prompt_tokens: int
    status: SequenceStatus
    temperature: float
    max_tokens: int
    stop_token_ids: FrozenSet[int]
    output_logprobs: List[float]

    def append_token(self, token_id: int, logprob: float) -> None:
        assert self.status == SequenceStatus.RUNNING
        self.token_ids.append(token_id)
        self.output_logprobs.append(logprob)

    @property
    def num_generated(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def is_finished(self) -> bool:
        return self.status == SequenceStatus.FINISHED

    def to_training_sample(self, weight_version: int) -> TrainingSample:
        assert self.status == SequenceStatus.FINISHED
        n = self.num_prompt_tokens
        stopped = self.token_ids[-1] in self.stop_token_ids
        return TrainingSample(
            prompt_tokens=tuple(self.token_ids[:n]),
            completion_tokens=tuple(self.token_ids[n:]),
            logprobs=tuple(self.output_logprobs),
            ref_logprobs=None,
            weight_version=weight_version,
            finish_reason="stop" if stopped else "length",
        )
