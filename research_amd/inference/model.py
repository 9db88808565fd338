"""Llama-style decoder whose attention runs on the paged backend.

The reference's engine loads a HuggingFace causal LM and recomputes the whole
sequence every step (rollouts/rollouts/inference/engine.py:60-68, :218-250);
its design puts an ``Attention(layer_idx, backend)`` module inside each block
(attention/layer.py:10-51, attention/example.py:45-96).  This is that block
structure for the Llama / Qwen2 family, stated after the reference's functional
Llama (rollouts/tools/functional_extractor/llama_functional.py: RMSNorm :50-65,
rotary tables :101-136, attention :160-225, SwiGLU MLP :228-247): parameter
names follow the HuggingFace checkpoint layout, so ``load_state_dict`` takes a
trainer's weights or a local safetensors checkpoint as they are.  Linear
layers, norms and the MLP are ordinary torch modules; the rotary embedding,
the KV append and attention go through ``Attention.forward_rope``.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Optional

import torch
from torch import Tensor, nn

from .attention import Attention, AttentionBackend
from .types import InferenceContext


@dataclass(frozen=True)
class ModelConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-5
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    attention_bias: bool = False  # Qwen2 checkpoints carry q/k/v biases

    @classmethod
    def from_hf_dict(cls, d: dict) -> "ModelConfig":
        """From the fields of a HuggingFace ``config.json`` of the Llama / Qwen2 family."""
        heads = d["num_attention_heads"]
        return cls(
            vocab_size=d["vocab_size"], hidden_size=d["hidden_size"], intermediate_size=d["intermediate_size"],
            num_layers=d["num_hidden_layers"], num_heads=heads, num_kv_heads=d.get("num_key_value_heads", heads),
            head_dim=d.get("head_dim") or d["hidden_size"] // heads, rope_theta=float(d.get("rope_theta", 10000.0)),
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),
            max_position_embeddings=int(d.get("max_position_embeddings", 8192)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            attention_bias=bool(d.get("attention_bias", d.get("model_type") == "qwen2")),
        )


class RMSNorm(nn.Module):
    def __init__(self, size: int, eps: float) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(size))
        self.eps = eps

    def forward(self, x: Tensor) -> Tensor:
        # statistics in float32, weight applied in the input type (llama_functional.py:61-65)
        xf = x.to(torch.float32)
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)
        return self.weight * xf.to(x.dtype)


class _SelfAttention(nn.Module):
    def __init__(self, cfg: ModelConfig, layer_idx: int, backend: AttentionBackend) -> None:
        super().__init__()
        self.cfg = cfg
        self.q_proj = nn.Linear(cfg.hidden_size, cfg.num_heads * cfg.head_dim, bias=cfg.attention_bias)
        self.k_proj = nn.Linear(cfg.hidden_size, cfg.num_kv_heads * cfg.head_dim, bias=cfg.attention_bias)
        self.v_proj = nn.Linear(cfg.hidden_size, cfg.num_kv_heads * cfg.head_dim, bias=cfg.attention_bias)
        self.o_proj = nn.Linear(cfg.num_heads * cfg.head_dim, cfg.hidden_size, bias=False)
        self.attn = Attention(layer_idx, backend)

    def forward(self, x: Tensor, cos: Tensor, sin: Tensor, positions: Tensor, ctx: InferenceContext) -> Tensor:
        b, t, _ = x.shape
        cfg = self.cfg
        q = self.q_proj(x).view(b, t, cfg.num_heads, cfg.head_dim)
        k = self.k_proj(x).view(b, t, cfg.num_kv_heads, cfg.head_dim)
        v = self.v_proj(x).view(b, t, cfg.num_kv_heads, cfg.head_dim)
        out = self.attn.forward_rope(q, k, v, cos, sin, ctx, positions=positions)
        return self.o_proj(out.reshape(b, t, cfg.num_heads * cfg.head_dim))


class _MLP(nn.Module):
    def __init__(self, cfg: ModelConfig) -> None:
        super().__init__()
        self.gate_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.up_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, bias=False)
        self.down_proj = nn.Linear(cfg.intermediate_size, cfg.hidden_size, bias=False)

    def forward(self, x: Tensor) -> Tensor:
        return self.down_proj(nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))


class _Block(nn.Module):
    def __init__(self, cfg: ModelConfig, layer_idx: int, backend: AttentionBackend) -> None:
        super().__init__()
        self.self_attn = _SelfAttention(cfg, layer_idx, backend)
        self.mlp = _MLP(cfg)
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)

    def forward(self, x: Tensor, cos: Tensor, sin: Tensor, positions: Tensor, ctx: InferenceContext) -> Tensor:
        x = x + self.self_attn(self.input_layernorm(x), cos, sin, positions, ctx)
        return x + self.mlp(self.post_attention_layernorm(x))


class _Trunk(nn.Module):
    def __init__(self, cfg: ModelConfig, backend: AttentionBackend) -> None:
        super().__init__()
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = nn.ModuleList(_Block(cfg, i, backend) for i in range(cfg.num_layers))
        self.norm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)


class PagedLlama(nn.Module):
    """``forward(input_ids [B, T], positions [B, T], ctx)`` -> hidden states ``[B, T, hidden]``;
    ``logits(hidden_rows)`` applies the final norm and the output projection to the rows that need them."""

    def __init__(self, cfg: ModelConfig, backend: AttentionBackend) -> None:
        super().__init__()
        self.cfg = cfg
        self.backend = backend
        backend.set_num_heads(cfg.num_heads)
        self.model = _Trunk(cfg, backend)
        self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False)
        if cfg.tie_word_embeddings:
            self.lm_head.weight = self.model.embed_tokens.weight
        self._rope = None  # (cos, sin) tables [max_position_embeddings, head_dim], built on first use

    def rope_tables(self, device, dtype):
        """cos / sin of ``position * theta**(-2i/D)``, both halves of a row alike, computed in float32 and
        cast once (llama_functional.py:101-136)."""
        if self._rope is None or self._rope[0].device != device or self._rope[0].dtype != dtype:
            cfg = self.cfg
            inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, device=device).float() / cfg.head_dim))
            angles = torch.arange(cfg.max_position_embeddings, device=device).float()[:, None] * inv_freq[None, :]
            emb = torch.cat((angles, angles), dim=-1)
            self._rope = (emb.cos().to(dtype).contiguous(), emb.sin().to(dtype).contiguous())
        return self._rope

    def forward(self, input_ids: Tensor, positions: Tensor, ctx: InferenceContext) -> Tensor:
        x = self.model.embed_tokens(input_ids)
        cos, sin = self.rope_tables(x.device, x.dtype)
        for block in self.model.layers:
            x = block(x, cos, sin, positions, ctx)
        return x

    def logits(self, hidden_rows: Tensor) -> Tensor:
        return self.lm_head(self.model.norm(hidden_rows))

    @classmethod
    def from_local(cls, path: str, backend_factory, dtype: torch.dtype = torch.bfloat16,
                   device: str = "cuda") -> "PagedLlama":
        """Build from a local HuggingFace checkpoint directory (``config.json`` + ``*.safetensors``); nothing is
        downloaded.  ``backend_factory(model_config)`` returns the attention backend to use."""
        from safetensors.torch import load_file

        with open(os.path.join(path, "config.json")) as fh:
            cfg = ModelConfig.from_hf_dict(json.load(fh))
        model = cls(cfg, backend_factory(cfg)).to(dtype)
        state = {}
        for name in sorted(os.listdir(path)):
            if name.endswith(".safetensors"):
                state.update(load_file(os.path.join(path, name)))
        if not state:
            raise FileNotFoundError(f"no .safetensors files in {path}")
        missing, unexpected = model.load_state_dict(state, strict=False)
        missing = [m for m in missing if not (cfg.tie_word_embeddings and m == "lm_head.weight")]
        if missing:
            raise RuntimeError(f"checkpoint lacks {missing[:5]}")
        return model.to(device).eval()


def default_num_kv_blocks(max_batch_size: int, max_model_len: int, block_size: int, cap: int = 65536) -> int:
    return min(cap, max_batch_size * (-(-max_model_len // block_size)))
