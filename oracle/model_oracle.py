"""CPU restatement of the model forward and of the reference engine's generation loop.  TEST INFRASTRUCTURE.

Nothing in the product imports this file.  It restates, with plain torch calls on the CPU and without importing
the reference:

* the Llama-family forward pass the reference's engine obtains from ``AutoModelForCausalLM``
  (rollouts/rollouts/inference/engine.py:60-68), following the reference's functional statement of it
  (rollouts/tools/functional_extractor/llama_functional.py:50-65 RMSNorm, :68-98 rotary embedding, :101-136
  tables, :160-225 attention with GQA and causal SDPA, :228-247 SwiGLU, :355-393 the stack);
* the engine's cache-less generation step (engine.py:218-250): every step feeds the whole token list, takes the
  last position's logits, samples, appends, and checks the stop conditions (engine.py:252-266).

How it is pinned (tests/test_oracle_model.py):
  llama_forward      equals ``transformers.LlamaForCausalLM`` (the class the reference's loader instantiates
                     for such checkpoints) on the same random weights, logits to 1e-5 in float32, with and
                     without grouped kv heads; causality: logits at position t do not depend on tokens after t
  generate_recompute greedy decoding is deterministic: equals repeated argmax of llama_forward by construction
                     of the loop; the loop's stop rules are checked on hand-made cases (stop token, max_tokens)
"""

from __future__ import annotations

from typing import Dict, FrozenSet, List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

from .paged_oracle import rope_literal, rope_tables


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Statistics in float32, weight applied in the input type (llama_functional.py:61-65)."""
    xf = x.to(torch.float32)
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return weight * xf.to(x.dtype)


def llama_forward(weights: Dict[str, torch.Tensor], cfg, input_ids: torch.Tensor) -> torch.Tensor:
    """Logits ``[B, T, vocab]`` of a full causal pass over ``input_ids [B, T]`` at positions 0..T-1.

    ``cfg`` needs num_layers, num_heads, num_kv_heads, head_dim, rope_theta, rms_norm_eps; ``weights`` uses the
    HuggingFace parameter names.
    """
    b, t = input_ids.shape
    x = F.embedding(input_ids, weights["model.embed_tokens.weight"])
    pos = torch.arange(t)[None].expand(b, -1)
    cos, sin = rope_tables(pos, cfg.head_dim, cfg.rope_theta, x.dtype)  # [B, T, D]
    cos, sin = cos.reshape(b * t, -1), sin.reshape(b * t, -1)
    n_rep = cfg.num_heads // cfg.num_kv_heads
    for i in range(cfg.num_layers):
        p = f"model.layers.{i}."
        h = rms_norm(x, weights[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        q = F.linear(h, weights[p + "self_attn.q_proj.weight"], weights.get(p + "self_attn.q_proj.bias"))
        k = F.linear(h, weights[p + "self_attn.k_proj.weight"], weights.get(p + "self_attn.k_proj.bias"))
        v = F.linear(h, weights[p + "self_attn.v_proj.weight"], weights.get(p + "self_attn.v_proj.bias"))
        q = rope_literal(q.view(b * t, cfg.num_heads, cfg.head_dim), cos, sin).view(b, t, cfg.num_heads, cfg.head_dim)
        k = rope_literal(k.view(b * t, cfg.num_kv_heads, cfg.head_dim), cos, sin).view(b, t, cfg.num_kv_heads, cfg.head_dim)
        v = v.view(b, t, cfg.num_kv_heads, cfg.head_dim)
        qt = q.transpose(1, 2)
        kt = k.transpose(1, 2).repeat_interleave(n_rep, dim=1)
        vt = v.transpose(1, 2).repeat_interleave(n_rep, dim=1)
        att = F.scaled_dot_product_attention(qt, kt, vt, is_causal=True)
        att = att.transpose(1, 2).reshape(b, t, cfg.num_heads * cfg.head_dim)
        x = x + F.linear(att, weights[p + "self_attn.o_proj.weight"])
        h = rms_norm(x, weights[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        gate = F.linear(h, weights[p + "mlp.gate_proj.weight"])
        up = F.linear(h, weights[p + "mlp.up_proj.weight"])
        x = x + F.linear(F.silu(gate) * up, weights[p + "mlp.down_proj.weight"])
    x = rms_norm(x, weights["model.norm.weight"], cfg.rms_norm_eps)
    head = weights.get("lm_head.weight", weights["model.embed_tokens.weight"])
    return F.linear(x, head)


def generate_recompute(weights: Dict[str, torch.Tensor], cfg, prompts: Sequence[Sequence[int]], max_tokens: int,
                       stop_token_ids: FrozenSet[int] = frozenset(), eos_token_id: Optional[int] = None
                       ) -> List[Tuple[List[int], List[float], str]]:
    """Greedy (temperature 0) generation the way the reference's engine steps without a KV cache
    (engine.py:218-266): per sequence and step, a full forward over all tokens so far, argmax of the last
    position, its log probability from the unscaled logits (sampling.py:31-33,:55).  Returns, per prompt,
    (completion tokens, log probabilities, finish reason)."""
    out = []
    for prompt in prompts:
        tokens = list(prompt)
        logprobs: List[float] = []
        while True:
            logits = llama_forward(weights, cfg, torch.tensor([tokens]))[:, -1].float()
            token = int(logits.argmax(dim=-1))
            logprobs.append(float(F.log_softmax(logits, dim=-1)[0, token]))
            tokens.append(token)
            generated = len(tokens) - len(prompt)
            if token in stop_token_ids or (eos_token_id is not None and token == eos_token_id) or generated >= max_tokens:
                break
        reason = "stop" if tokens[-1] in stop_token_ids else "length"
        out.append((tokens[len(prompt):], logprobs, reason))
    return out


def logprobs_of(weights: Dict[str, torch.Tensor], cfg, tokens: Sequence[int], num_prompt_tokens: int) -> List[float]:
    """Log probability of every completion token of ``tokens`` given everything before it (one full pass)."""
    logits = llama_forward(weights, cfg, torch.tensor([list(tokens)])).float()
    lp = F.log_softmax(logits[0, num_prompt_tokens - 1 : -1], dim=-1)
    want = torch.tensor(list(tokens[num_prompt_tokens:]))
    return lp.gather(-1, want[:, None])[:, 0].tolist()
