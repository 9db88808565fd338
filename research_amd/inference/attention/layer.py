"""``nn.Module`` shim that a transformer block holds in place of attention math.

Same constructor and call signature as the reference's ``Attention``
(rollouts/rollouts/inference/attention/layer.py:10-51): no parameters, it
remembers which layer it is and forwards to the shared backend.
"""

from __future__ import annotations

from torch import Tensor, nn

from ..types import InferenceContext
from .protocol import AttentionBackend


class Attention(nn.Module):
    def __init__(self, layer_idx: int, backend: AttentionBackend) -> None:
        super().__init__()
        self.layer_idx = layer_idx
        self.backend = backend

    def forward(self, q: Tensor, k: Tensor, v: Tensor, ctx: InferenceContext) -> Tensor:
        return self.backend.forward(q, k, v, self.layer_idx, ctx)

    def forward_rope(self, q: Tensor, k: Tensor, v: Tensor, cos: Tensor, sin: Tensor, ctx: InferenceContext,
                     positions=None) -> Tensor:
        """``forward`` on rotary-embedded q and k with the rotation fused into the KV append (an addition: the
        reference's blocks rotate q and k themselves, llama_functional.py:203, and then call ``forward``)."""
        return self.backend.forward_rope(q, k, v, cos, sin, self.layer_idx, ctx, positions=positions)
