"""Per-step descriptor handed to every attention layer.

Mirrors the field names, order and defaults of the reference's
``InferenceContext`` (rollouts/rollouts/inference/types.py:72-107) so that
code which builds a context for the reference backend builds one for this
backend unchanged.  Only the type that the attention / KV-cache path consumes
is restated here; the engine, sampling and scheduler dataclasses of the same
reference file are not on that path.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


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
    ``block_mask``    opaque mask object; this backend accepts ``None`` only.

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
