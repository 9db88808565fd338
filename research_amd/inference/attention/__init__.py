"""Attention over a paged KV pool (reference: rollouts/rollouts/inference/attention/__init__.py).

``FlexAttentionBackend`` is kept as an alias of ``HipPagedAttentionBackend`` so
that ``from ...attention import CacheConfig, FlexAttentionBackend`` keeps working.
"""

from .config import CacheConfig
from .hip_backend import FlexAttentionBackend, HipPagedAttentionBackend
from .layer import Attention
from .protocol import AttentionBackend

__all__ = ["CacheConfig", "AttentionBackend", "HipPagedAttentionBackend", "FlexAttentionBackend", "Attention"]
