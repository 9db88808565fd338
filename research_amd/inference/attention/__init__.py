"""Attention over a paged KV pool (reference: rollouts/rollouts/inference/attention/__init__.py).

``FlexAttentionBackend`` is ``HipPagedAttentionBackend`` with the reference's decode numerics as
defaults, so that ``from ...attention import CacheConfig, FlexAttentionBackend`` keeps working and
keeps its results.
"""

from .config import CacheConfig
from .hip_backend import FlexAttentionBackend, HipPagedAttentionBackend
from .layer import Attention
from .mask import (PagedMask, create_attention_mask, create_causal_block_mask, create_document_mask,
                   create_sliding_window_causal_mask)
from .protocol import AttentionBackend

_BACKEND = ("Attention", "AttentionBackend", "CacheConfig", "FlexAttentionBackend", "HipPagedAttentionBackend")
_MASKS = ("PagedMask", "create_attention_mask", "create_causal_block_mask", "create_document_mask",
          "create_sliding_window_causal_mask")
__all__ = [*_BACKEND, *_MASKS]
