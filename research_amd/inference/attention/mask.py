"""Attention masks for the paged kernels (reference: rollouts/rollouts/inference/attention/mask.py).

The reference builds FlexAttention ``BlockMask`` objects from a per-entry
predicate.  The HIP kernels do not evaluate predicates: every mask the
reference offers restricts a query row to one contiguous key range
``first_key(row) <= kv_idx <= q_idx``, so a mask here is a small frozen
description of that range which the backend turns into kernel arguments:

* causal (mask.py:20-53)                     -> nothing to pass,
* causal sliding window (mask.py:56-100)     -> the ``window`` argument,
* packed documents (mask.py:141-191)         -> one first key per query row.

The factory functions keep the reference's names, parameters and defaults.
``block_size`` and ``device`` are accepted and ignored: there is no block
structure to precompute and nothing lives on a device until a step uses it.
``mask_mod`` evaluates the reference's predicate for one entry, which is what
the tests compare the kernels' range form with.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import numpy as np


@dataclass(frozen=True)
class PagedMask:
    """Key range of every query row: ``max(q - window + 1, start of q's document) <= kv <= q``.

    ``window``: sliding window or None.  ``boundaries``: document starts plus the
    final end, as running sums of the document lengths (mask.py:168-171), or None.
    """

    batch_size: int
    seq_len: int
    window: Optional[int] = None
    boundaries: Optional[Tuple[int, ...]] = None

    @property
    def kind(self) -> str:
        if self.boundaries is not None:
            return "document"
        return "sliding_window" if self.window is not None else "causal"

    def mask_mod(self, b: int, h: int, q_idx: int, kv_idx: int) -> bool:
        """The reference predicate of this mask for one (query, key) entry."""
        keep = q_idx >= kv_idx  # mask.py:42-43
        if self.window is not None:
            keep = keep and (q_idx - kv_idx) < self.window  # mask.py:83-89
        if self.boundaries is not None:  # mask.py:173-186
            q_doc = sum(1 for end in self.boundaries[1:] if q_idx >= end)
            kv_doc = sum(1 for end in self.boundaries[1:] if kv_idx >= end)
            keep = keep and q_doc == kv_doc
        return bool(keep)

    def first_keys(self, positions: np.ndarray) -> np.ndarray:
        """First key (int32) that the rows at ``positions`` attend under the document part of the mask."""
        positions = np.asarray(positions, dtype=np.int64)
        if self.boundaries is None:
            return np.zeros(positions.shape, dtype=np.int32)
        bounds = np.asarray(self.boundaries, dtype=np.int64)
        doc = np.searchsorted(bounds[1:], positions, side="right")  # number of document ends <= position
        return bounds[doc].astype(np.int32)


def create_causal_block_mask(batch_size: int, seq_len: int, block_size: int = 128, device="cuda") -> PagedMask:
    """Causal mask (mask.py:20-53)."""
    return PagedMask(batch_size=batch_size, seq_len=seq_len)


def create_sliding_window_causal_mask(batch_size: int, seq_len: int, window_size: int, block_size: int = 128,
                                      device="cuda") -> PagedMask:
    """Causal mask with a sliding window: ``q_idx >= kv_idx`` and ``q_idx - kv_idx < window_size`` (mask.py:56-100)."""
    if window_size <= 0:
        raise ValueError(f"window_size={window_size} must be positive")
    return PagedMask(batch_size=batch_size, seq_len=seq_len, window=int(window_size))


def create_attention_mask(batch_size: int, seq_len: int, sliding_window: Optional[int] = None, block_size: int = 128,
                          device="cuda") -> PagedMask:
    """Sliding-window mask when ``sliding_window`` is set, else causal (mask.py:103-138)."""
    if sliding_window is not None:
        return create_sliding_window_causal_mask(batch_size=batch_size, seq_len=seq_len, window_size=sliding_window,
                                                 block_size=block_size, device=device)
    return create_causal_block_mask(batch_size=batch_size, seq_len=seq_len, block_size=block_size, device=device)


def create_document_mask(batch_size: int, seq_lens: Tuple[int, ...], total_len: int, block_size: int = 128,
                         device="cuda") -> PagedMask:
    """Causal attention inside each of the documents packed into a row of ``total_len`` tokens (mask.py:141-191).

    Document i covers positions ``[sum(seq_lens[:i]), sum(seq_lens[:i+1]))``; positions past the last
    document form one more document, as the reference's predicate has it.
    """
    bounds = [0]
    for length in seq_lens:
        if length < 0:
            raise ValueError("document lengths must be non-negative")
        bounds.append(bounds[-1] + int(length))
    return PagedMask(batch_size=batch_size, seq_len=total_len, boundaries=tuple(bounds))
