"""Attention / KV-cache call surface (reference: rollouts/rollouts/inference/__init__.py).

Exports the subset of the reference package's names that belong to the paged
attention path; the engine, scheduler and sampling names are not part of it.
"""

from .attention import Attention, AttentionBackend, CacheConfig, FlexAttentionBackend, HipPagedAttentionBackend
from .cache import PagedKVCache
from .context import (
    allocate_and_build_context,
    build_chunked_prefill_context,
    build_decode_context,
    build_prefill_context,
    extend_and_build_context,
)
from .types import InferenceContext

__all__ = [
    "InferenceContext",
    "CacheConfig",
    "build_prefill_context",
    "build_decode_context",
    "build_chunked_prefill_context",
    "allocate_and_build_context",
    "extend_and_build_context",
    "AttentionBackend",
    "HipPagedAttentionBackend",
    "FlexAttentionBackend",
    "Attention",
    "PagedKVCache",
]
