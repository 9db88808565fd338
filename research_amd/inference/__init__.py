"""Inference package on the paged attention path (reference: rollouts/rollouts/inference/__init__.py).

Exports the reference package's names: the attention / KV-cache call surface and the engine, scheduler and
sampling that drive it.
"""

from .attention import (Attention, AttentionBackend, CacheConfig, FlexAttentionBackend, HipPagedAttentionBackend,
                        create_causal_block_mask)
from .cache import PagedKVCache, RadixKVCache
from .context import (allocate_and_build_context, build_chunked_prefill_context, build_decode_context,
                      build_prefill_context, extend_and_build_context)
from .engine import InferenceEngine
from .model import ModelConfig, PagedLlama
from .sampling import sample_with_logprobs
from .scheduler import schedule
from .types import (EngineConfig, InferenceContext, SamplingParams, SchedulerConfig, SchedulerOutput, Sequence,
                    SequenceStatus, TrainingSample)

# What the package exports, by the part of the path it belongs to (alphabetical inside a group).
_ATTENTION = ("Attention", "AttentionBackend", "CacheConfig", "FlexAttentionBackend", "HipPagedAttentionBackend",
              "create_causal_block_mask")
_ALLOCATORS = ("PagedKVCache", "RadixKVCache")
_CONTEXTS = ("InferenceContext", "allocate_and_build_context", "build_chunked_prefill_context",
             "build_decode_context", "build_prefill_context", "extend_and_build_context")
_ENGINE = ("EngineConfig", "InferenceEngine", "ModelConfig", "PagedLlama", "SamplingParams", "SchedulerConfig",
           "SchedulerOutput", "Sequence", "SequenceStatus", "TrainingSample", "sample_with_logprobs", "schedule")
__all__ = [*_ATTENTION, *_ALLOCATORS, *_CONTEXTS, *_ENGINE]
