"""Sampling as pure functions over logits (reference: rollouts/rollouts/inference/sampling.py).

Tokens are drawn from the temperature-scaled distribution; the reported log
probabilities always come from the unscaled logits, i.e. the model's own
distribution, which is what an RL trainer needs.
"""

from __future__ import annotations

from typing import Tuple

import torch
import torch.nn.functional as F
from torch import Tensor


def sample_with_logprobs(logits: Tensor, temperatures: Tensor) -> Tuple[Tensor, Tensor]:
    """``logits [batch, vocab]``, ``temperatures [batch]`` -> sampled ids and their log probabilities
    (sampling.py:11-59).  Temperature 0 selects the argmax."""
    assert logits.dim() == 2, f"Expected 2D logits, got {logits.dim()}D"
    assert temperatures.dim() == 1, f"Expected 1D temperatures, got {temperatures.dim()}D"
    assert logits.size(0) == temperatures.size(0), "Batch size mismatch"
    greedy = temperatures == 0
    divisor = torch.where(greedy, torch.ones_like(temperatures), temperatures)
    probs = F.softmax(logits / divisor.unsqueeze(-1), dim=-1)
    tokens = torch.multinomial(probs, num_samples=1).squeeze(-1)
    tokens = torch.where(greedy, logits.argmax(dim=-1), tokens)
    logprobs = F.log_softmax(logits, dim=-1).gather(-1, tokens.unsqueeze(-1)).squeeze(-1)
    return tokens, logprobs


def sample_greedy(logits: Tensor) -> Tuple[Tensor, Tensor]:
    """Argmax ids and their log probabilities (sampling.py:62-79)."""
    assert logits.dim() == 2
    tokens = logits.argmax(dim=-1)
    return tokens, F.log_softmax(logits, dim=-1).gather(-1, tokens.unsqueeze(-1)).squeeze(-1)


def compute_logprobs_for_tokens(logits: Tensor, tokens: Tensor) -> Tensor:
    """Log probability of ``tokens [batch, seq]`` under ``logits [batch, seq, vocab]`` (sampling.py:82-103)."""
    assert logits.dim() == 3
    assert tokens.dim() == 2
    assert logits.shape[:2] == tokens.shape
    return F.log_softmax(logits, dim=-1).gather(-1, tokens.unsqueeze(-1)).squeeze(-1)
