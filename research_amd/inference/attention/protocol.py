"""Structural interface every attention backend satisfies.

Restates the single-method protocol of the reference
(rollouts/rollouts/inference/attention/protocol.py:10-40): a backend owns the
KV pool for all layers and is handed ``layer_idx`` to pick its slice.
"""

from __future__ import annotations

from typing import Protocol, runtime_checkable

from torch import Tensor

from ..types import InferenceContext


@runtime_checkable
class AttentionBackend(Protocol):
    def forward(
        self,
        q: Tensor,  # [batch, seq_len, num_heads, head_dim]
        k: Tensor,  # [batch, seq_len, num_kv_heads, head_dim]
        v: Tensor,  # [batch, seq_len, num_kv_heads, head_dim]
        layer_idx: int,
        ctx: InferenceContext,
    ) -> Tensor:  # [batch, seq_len, num_heads, head_dim]
        ...
