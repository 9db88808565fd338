"""Paged-KV attention backend for MI355X behind the reference's call surface.

``HipPagedAttentionBackend`` has the constructor, attributes and methods of
the reference's ``FlexAttentionBackend``
(rollouts/rollouts/inference/attention/flex_backend.py:11-285) and can stand in
for it inside an ``Attention`` layer.  Where the reference issues PyTorch
indexing / ``scaled_dot_product_attention`` calls, this class passes raw device
pointers of the same tensors to the C ABI of ``libpaged_attn.so``; torch is used
for device memory and the current stream only.  There is no eager fallback: a
missing library, or tensors that are not on a HIP device, raise.

Two classes: ``HipPagedAttentionBackend`` defaults to exact-length, windowed
decode (the first and third points below); ``FlexAttentionBackend``, the
reference's name, is the same class with the reference's decode numerics as
defaults (``pad_zero_keys=True, window_in_decode=False``), so code that imports
it by that name gets the reference's results on ragged batches too.

Differences of ``HipPagedAttentionBackend`` from the reference, all deliberate:

* Decode attends exactly ``seq_lens[b]`` keys per sequence.  The reference
  zero-pads a ragged batch to its longest sequence and attends without a mask
  (flex_backend.py:253-264, :227-229), which lets the padding keys (logit 0)
  take softmax mass; the two agree whenever all lengths are equal (always for
  batch 1).  ``pad_zero_keys=True`` reproduces the reference's ragged result.
* ``ctx.prefix_lens`` (an added, optional context field) selects chunked
  prefill: the chunk's queries attend the cached prefix and the chunk itself,
  both read from the pool through the block table.
* ``config.sliding_window`` is applied inside the kernels (a row at position p
  sees keys ``p - window < j <= p``, attention/mask.py:83-89) instead of through
  a FlexAttention ``BlockMask``; ``get_block_mask`` returns the ``PagedMask``
  description of it (``None`` without a window, as in the reference).
  Prefill applies it as the reference does.  Decode in the reference applies a
  window only when the caller passes ``ctx.block_mask`` (flex_backend.py:220-225)
  and otherwise attends the whole cache; ``window_in_decode=False`` keeps that,
  the default ``True`` attends the last ``window`` keys, consistent with prefill.
* ``ctx.block_mask`` takes the ``PagedMask`` objects of ``attention/mask.py``
  (causal, sliding window, packed documents): a window becomes the kernels'
  ``window`` argument and documents become one first key per query row.  A
  ``mask_mod(b, h, q_idx, kv_idx)`` callable, or an object that carries one (a
  FlexAttention ``BlockMask``), is evaluated once per context, packed into bits
  and applied by the general masked kernel.  Anything else raises
  ``NotImplementedError`` instead of being ignored.  A document mask describes
  packed prefill rows; in decode it raises.
"""

from __future__ import annotations

from collections import OrderedDict
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch
from torch import Tensor

from ... import _lib, ops
from ..types import InferenceContext
from .config import CacheConfig
from .mask import PagedMask, create_attention_mask

_COMPUTE_DTYPES = (torch.float32, torch.bfloat16, torch.float16)


class _StepTensors:
    """Device copies of one context's integer fields, built once per step."""

    __slots__ = ("ctx", "slots", "touched", "tables", "bt_stride", "seq_lens", "extra_zero", "ctx_lens", "q_lens",
                 "q_starts", "max_q_len", "row_first_key", "fp8_blocks", "fp8_tables", "mask_words", "mask_keys")

    def __init__(self, ctx: InferenceContext) -> None:
        self.ctx = ctx  # keeps id(ctx) alive while the entry is cached
        self.slots = self.touched = self.tables = self.seq_lens = self.extra_zero = None
        self.ctx_lens = self.q_lens = self.q_starts = self.row_first_key = None
        self.fp8_blocks = self.fp8_tables = None  # distinct blocks of the tables and the tables renumbered to them
        self.mask_words = None  # bits of an arbitrary mask predicate evaluated for this step, and their key count
        self.mask_keys = 0
        self.bt_stride = self.max_q_len = 0


def _padded_tables(block_tables: Sequence[Sequence[int]]) -> np.ndarray:
    width = max((len(row) for row in block_tables), default=0)
    out = np.full((len(block_tables), max(width, 1)), -1, dtype=np.int32)
    for i, row in enumerate(block_tables):
        if len(row):
            out[i, : len(row)] = np.asarray(row, dtype=np.int64)
    return out


class HipPagedAttentionBackend:
    _mask_round_elems = 1 << 28  # (sequence, head, row, key) entries of a mask predicate evaluated per round

    def __init__(self, config: CacheConfig, pad_zero_keys: bool = False, window_in_decode: bool = True) -> None:
        self._lib = _lib.load()  # raises if the HIP library has not been built
        self.config = config
        self.num_heads_per_kv = 1  # until set_num_heads(), as in the reference (flex_backend.py:31,43-45)
        self.scale = config.head_dim**-0.5
        self.pad_zero_keys = pad_zero_keys
        if config.sliding_window is not None and config.sliding_window <= 0:
            raise ValueError(f"sliding_window={config.sliding_window} must be positive")
        self._window = int(config.sliding_window or 0)
        self.window_in_decode = window_in_decode
        if self._window and pad_zero_keys and window_in_decode:
            raise ValueError("pad_zero_keys cannot be combined with a sliding window in decode")
        self._mask_cache: dict = {}
        self._step_cache: "OrderedDict[int, _StepTensors]" = OrderedDict()
        self._workspace: Optional[Tensor] = None
        self._retired_workspaces: List[Tensor] = []

        if config.kv_format not in (None, "fp8_e4m3"):
            raise ValueError(f"unknown kv_format {config.kv_format!r}")
        if config.dtype not in _COMPUTE_DTYPES:
            raise ValueError(f"unsupported cache dtype {config.dtype}")
        self._fp8 = config.kv_format == "fp8_e4m3"
        pool_dtype = torch.float8_e4m3fn if self._fp8 else config.dtype
        # one allocation per tensor for all layers, zero-initialised (flex_backend.py:38-41)
        self.k_cache = torch.zeros(config.cache_shape, dtype=pool_dtype, device=config.device)
        self.v_cache = torch.zeros(config.cache_shape, dtype=pool_dtype, device=config.device)
        self.k_scale = self.v_scale = None
        if self._fp8:
            shape = (config.num_layers, config.num_blocks, config.num_kv_heads)
            self.k_scale = torch.ones(shape, dtype=torch.float32, device=config.device)
            self.v_scale = torch.ones(shape, dtype=torch.float32, device=config.device)

    # ------------------------------------------------------------------ small surface
    def set_num_heads(self, num_heads: int) -> None:
        self.num_heads_per_kv = num_heads // self.config.num_kv_heads

    def get_block_mask(self, batch_size: int, seq_len: int) -> object:
        """The configured mask for a step of this shape (flex_backend.py:47-83): ``None`` for plain causal,
        else the sliding-window description, cached per shape with the reference's bound of 100 entries."""
        if self.config.sliding_window is None:
            return None
        key = (batch_size, seq_len)
        mask = self._mask_cache.get(key)
        if mask is None:
            mask = create_attention_mask(batch_size=batch_size, seq_len=seq_len,
                                         sliding_window=self.config.sliding_window,
                                         block_size=self.config.block_size, device=self.config.device)
            if len(self._mask_cache) < 100:
                self._mask_cache[key] = mask
        return mask

    def _mask_window(self, mask: object, default: int) -> int:
        """The ``window`` kernel argument under ``ctx.block_mask`` (which replaces the configured mask, as in
        flex_backend.py:170-173)."""
        if mask is None:
            return default
        if not isinstance(mask, PagedMask):
            raise NotImplementedError(
                f"block_mask of type {type(mask).__name__}: the HIP backend takes the PagedMask objects of "
                "attention/mask.py (causal, sliding window, documents), a mask_mod(b, h, q_idx, kv_idx) callable "
                "or an object that carries one (a FlexAttention BlockMask)")
        return int(mask.window or 0)

    @staticmethod
    def _mask_predicate(mask: object):
        """The ``mask_mod(b, h, q_idx, kv_idx)`` predicate of a mask that is not a ``PagedMask``: the object
        itself when callable, or its ``mask_mod`` attribute (what a FlexAttention ``BlockMask`` built by
        ``create_block_mask`` carries; the reference passes such objects to ``flex_attention``,
        flex_backend.py:170-178, :220-225).  None for ``None`` and for ``PagedMask`` objects, which the kernels
        apply themselves."""
        if mask is None or isinstance(mask, PagedMask):
            return None
        mod = getattr(mask, "mask_mod", None)
        if callable(mod):
            return mod
        return mask if callable(mask) else None

    def _mask_bits(self, step: _StepTensors, mod, batch: int, heads: int, q_pos: Tensor, n_keys: int) -> Tensor:
        """The predicate evaluated on every (sequence, head, row, key) of the step, packed into the words
        ``pa_attend_masked`` takes; computed once per context (all layers share it).  ``q_pos`` int ``[B, T]``:
        the q_idx of every row.  A predicate that does not look at ``h`` gives one row of bits for all heads."""
        if step.mask_words is None:
            dev = self.k_cache.device
            b = torch.arange(batch, device=dev)[:, None, None, None]
            h = torch.arange(heads, device=dev)[None, :, None, None]
            kv = torch.arange(n_keys, device=dev)[None, None, None, :]
            q_pos = q_pos.to(dev)
            rows_per_seq = q_pos.shape[1]
            # a bounded number of query rows at a time: the dense boolean result of one round stays near 256 MiB
            # even when the predicate looks at the head (a whole 8192-row step would be gigabytes)
            chunk = max(1, self._mask_round_elems // max(1, batch * heads * max(n_keys, 1)))
            parts = []
            for at in range(0, rows_per_seq, chunk):
                qi = q_pos[:, None, at: at + chunk, None]
                keep = torch.as_tensor(mod(b, h, qi, kv), device=dev).to(torch.bool)
                while keep.dim() < 4:
                    keep = keep[None]
                keep = keep.expand(batch, keep.shape[1], qi.shape[2], n_keys)  # one head when `h` is not looked at
                parts.append(ops.pack_mask(keep.permute(0, 2, 1, 3).reshape(batch * qi.shape[2], keep.shape[1], n_keys)))
            words = parts[0].shape[-1]
            if len(parts) == 1:
                packed = parts[0]
            else:  # rows of a sequence are contiguous in the step: interleave the rounds back into that order
                packed = torch.cat([p.view(batch, -1, p.shape[1], words) for p in parts], dim=1)
                packed = packed.reshape(batch * rows_per_seq, -1, words).contiguous()
            step.mask_words, step.mask_keys = packed, n_keys
        return step.mask_words

    def _mask_first_keys(self, mask: object, step: _StepTensors, batch: int, seq_len: int,
                         prefix: Optional[np.ndarray]) -> Optional[Tensor]:
        """Per-row first keys (int32 ``[batch * seq_len]``) of a document mask, None for the other masks.
        Row t of sequence b sits at position ``prefix[b] + t``."""
        if not isinstance(mask, PagedMask) or mask.boundaries is None:
            return None
        if step.row_first_key is None:
            pos = np.arange(seq_len, dtype=np.int64)[None, :] + (
                prefix[:, None] if prefix is not None else np.zeros((batch, 1), dtype=np.int64))
            step.row_first_key = self._to_device(np.ascontiguousarray(mask.first_keys(pos)).reshape(-1))
        return step.row_first_key

    def clear_mask_cache(self) -> None:
        self._mask_cache.clear()

    def clear_cache(self) -> None:
        self.k_cache.zero_()
        self.v_cache.zero_()
        if self._fp8:
            self.k_scale.fill_(1.0)
            self.v_scale.fill_(1.0)
        self._mask_cache.clear()
        self._step_cache.clear()

    # ------------------------------------------------------------------ forward
    def forward(self, q: Tensor, k: Tensor, v: Tensor, layer_idx: int, ctx: InferenceContext) -> Tensor:
        """Append this step's K/V, then attend (flex_backend.py:89-114).

        The append runs first, so a decode step sees its own token.
        """
        if ctx.slot_mapping is not None:
            self._store_kv(k, v, layer_idx, ctx.slot_mapping, _step=self._step(ctx), _ctx=ctx)
        return self._attend(q, k, v, layer_idx, ctx)

    __call__ = forward

    def _attend(self, q: Tensor, k: Tensor, v: Tensor, layer_idx: int, ctx: InferenceContext) -> Tensor:
        if ctx.is_prefill:
            if getattr(ctx, "prefix_lens", None) is not None:  # absent on the reference's own context type
                return self._prefill_paged(q, layer_idx, ctx)
            return self._prefill_attention(q, k, v, ctx)
        return self._decode_attention(q, layer_idx, ctx)

    def forward_rope(self, q: Tensor, k: Tensor, v: Tensor, cos: Tensor, sin: Tensor, layer_idx: int,
                     ctx: InferenceContext, positions: Optional[Tensor] = None) -> Tensor:
        """``forward`` on the rotary-embedded q and k, with the rotation fused into the KV append.

        Equals ``q, k = apply_rotary_pos_emb(q, k, cos, sin)`` (rollouts/tools/functional_extractor/
        llama_functional.py:75-98, evaluated in the tensors' dtype) followed by ``forward(q, k, v, layer_idx,
        ctx)``, but the new K rows are read once and written once: one kernel rotates q and k and writes the
        rotated k and v to their slots.  q ``[B, T, Hq, D]``, k/v ``[B, T, Hkv, D]``; cos/sin ``[B, T, D]`` (one
        row per token) or, with ``positions`` (int ``[B, T]``), a table ``[rows, D]`` indexed by position.
        q and k are not modified.
        """
        cfg = self.config
        batch, seq_len, num_heads, head_dim = q.shape
        n = batch * seq_len
        self._require_device(q, k, v, cos, sin, self.k_cache)
        q3 = q.contiguous().view(n, num_heads, head_dim)
        k3 = k.reshape(n, cfg.num_kv_heads, head_dim).contiguous()
        v3 = v.reshape(n, cfg.num_kv_heads, head_dim).contiguous()
        cos2 = cos.reshape(-1, head_dim).contiguous()
        sin2 = sin.reshape(-1, head_dim).contiguous()
        pos = None
        if positions is not None:
            pos = positions.reshape(-1).to(device=q.device, dtype=torch.int32).contiguous()
            if pos.numel() != n:
                raise ValueError("positions must hold one entry per token")
        elif cos2.shape[0] != n:
            raise ValueError("cos / sin must hold one row per token when no positions are given")
        q_rot = torch.empty_like(q3)
        if n == 0:
            return q_rot.view(q.shape)
        slots = None
        if ctx.slot_mapping is not None:
            step = self._step(ctx)
            slots = self._device_slots(ctx.slot_mapping, n, step)
        dense = ctx.is_prefill and getattr(ctx, "prefix_lens", None) is None  # attends the step's own K/V
        kc, vc = self._layer(layer_idx)
        if self._fp8 and slots is not None:
            self._touched(step, slots, ctx, layer_idx)
        if self._fp8 and slots is not None and not dense:
            ops.rope_kv_append_e4m3(q3, k3, v3, cos2, sin2, kc, vc, self.k_scale[layer_idx], self.v_scale[layer_idx],
                                    slots, cfg.block_size, positions=pos, q_out=q_rot, touched=step.touched)
            k_rot = None
        else:
            to_pool = slots is not None and not self._fp8  # rows of the pool's own type go straight to their slots
            if to_pool and k3.dtype != self.k_cache.dtype:
                raise RuntimeError("Index put requires the source and destination dtypes match")
            k_rot = torch.empty_like(k3) if dense or not to_pool else None
            ops.rope_kv_append(q3, k3, v3, cos2, sin2, kc if to_pool else None, vc if to_pool else None,
                               slots if to_pool else None, positions=pos, q_out=q_rot, k_out=k_rot)
            if self._fp8 and slots is not None:  # dense prefill keeps the rotated K: append it from there
                ops.kv_append_e4m3(kc, vc, self.k_scale[layer_idx], self.v_scale[layer_idx], k_rot, v3, slots,
                                   cfg.block_size, step.touched)
        k_att = k_rot.view(batch, seq_len, cfg.num_kv_heads, head_dim) if k_rot is not None else k
        return self._attend(q_rot.view(q.shape), k_att, v, layer_idx, ctx)

    # ------------------------------------------------------------------ helpers
    def _require_device(self, *tensors: Tensor) -> torch.device:
        for t in tensors:
            if t.device.type != "cuda":
                raise RuntimeError(
                    "HipPagedAttentionBackend computes only on a HIP device; "
                    f"got a tensor on {t.device} (there is no CPU implementation)"
                )
        return tensors[0].device

    def _step(self, ctx: InferenceContext) -> _StepTensors:
        key = id(ctx)
        hit = self._step_cache.get(key)
        if hit is not None and hit.ctx is ctx:
            self._step_cache.move_to_end(key)
            return hit
        entry = _StepTensors(ctx)
        self._step_cache[key] = entry
        while len(self._step_cache) > 4:
            self._step_cache.popitem(last=False)
        return entry

    def _to_device(self, array: np.ndarray) -> Tensor:
        return torch.from_numpy(array).to(self.k_cache.device)

    def _tables(self, step: _StepTensors, block_tables) -> None:
        """Device copy of the block tables.  The reference's tuple-of-tuples costs a Python-level pass over every
        block id (tens of ms at 256 sequences x 2000 blocks); a 2-D int32 array or tensor padded with -1 is
        taken as it is."""
        if step.tables is None:
            if isinstance(block_tables, Tensor):
                if block_tables.dim() != 2:
                    raise ValueError("block_tables tensor must be [num_seqs, width], padded with -1")
                if block_tables.device.type == "cuda":
                    # used as it is: a caller that rewrites it in place between graph replays must be read live
                    if block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
                        raise TypeError("a device-resident block_tables must be a contiguous int32 tensor")
                    step.tables = block_tables
                else:
                    step.tables = block_tables.to(device=self.k_cache.device, dtype=torch.int32).contiguous()
            elif isinstance(block_tables, np.ndarray):
                if block_tables.ndim != 2:
                    raise ValueError("block_tables array must be [num_seqs, width], padded with -1")
                step.tables = self._to_device(np.ascontiguousarray(block_tables, dtype=np.int32))
            else:
                step.tables = self._to_device(_padded_tables(block_tables))
            step.bt_stride = step.tables.shape[1]

    def _lens(self, values, batch: int) -> np.ndarray:
        """Host int64 copy of a per-sequence integer field (tuple, array or tensor)."""
        if isinstance(values, Tensor):
            values = values.detach().cpu().numpy()
        return np.asarray(values, dtype=np.int64)[:batch]

    def _workspace_for(self, nbytes: int) -> Tensor:
        """The decode workspace, grown on demand.  A buffer that has been handed out is never released while the
        backend lives: a captured graph of a decode step keeps replaying with the address it was recorded with,
        so an outgrown buffer is retired, not freed (growth at least doubles, which bounds what is retained)."""
        if self._workspace is None or self._workspace.numel() < nbytes:
            have = 0
            if self._workspace is not None:
                have = self._workspace.numel()
                self._retired_workspaces.append(self._workspace)
            # zero-filled: the arrival counters at the start of a workspace must read zero before its first use
            self._workspace = torch.zeros(max(nbytes, 2 * have, 1 << 20), dtype=torch.uint8,
                                          device=self.k_cache.device)
        return self._workspace

    def _layer(self, layer_idx: int) -> Tuple[Tensor, Tensor]:
        return self.k_cache[layer_idx], self.v_cache[layer_idx]

    def _device_slots(self, slot_mapping, n: int, step: Optional[_StepTensors], *tensors: Tensor) -> Tensor:
        """int64 device copy of a slot mapping (cached on the step), with the reference's error for a slot
        past the pool."""
        cfg = self.config
        if len(slot_mapping) != n:
            raise IndexError(
                f"The shape of the mask [{len(slot_mapping)}] at index 0 does not match the shape of the indexed "
                f"tensor [{n}, {cfg.num_kv_heads}, {cfg.head_dim}] at index 0")
        if step is not None and step.slots is not None:
            return step.slots
        if isinstance(slot_mapping, Tensor) and slot_mapping.device.type == "cuda":
            # already on the device: used as it is (out-of-range slots are dropped by the kernel, not reported)
            self._require_device(*tensors, self.k_cache)
            if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous():
                raise TypeError("a device-resident slot_mapping must be a contiguous int64 tensor")
            slots = slot_mapping
        else:
            if isinstance(slot_mapping, Tensor):
                slot_mapping = slot_mapping.numpy()
            host = np.asarray(slot_mapping, dtype=np.int64)
            if host.size and host.max() >= cfg.total_slots:
                raise IndexError(
                    f"index {int(host.max())} is out of bounds for dimension 0 with size {cfg.total_slots}")
            self._require_device(*tensors, self.k_cache)
            slots = self._to_device(host)
        if step is not None:
            step.slots = slots
        return slots

    # ------------------------------------------------------------------ KV append
    def _touched(self, step: Optional[_StepTensors], slots: Tensor, ctx: Optional[InferenceContext],
                 layer_idx: int):
        """The blocks an fp8 append works on (one workgroup each; entries outside the pool are skipped by the
        kernel): an ``ops.TouchedBlocks`` (distinct blocks and the index of the step's rows by block), or a bare
        int32 device list.

        A decode step whose slot mapping lives on the device writes one row per sequence, and every sequence
        writes into a block of its own, so the list is simply each slot's block (-1 for a padding row's slot
        -1): two device operations with no data-dependent shape and no host round trip, which a graph capture
        can record.  It is rebuilt at the first layer of every pass, so a pass recorded after an eager warm-up
        on the same context object contains it (no row index: with one row per sequence the kernel's scan of
        the slot list is short).  Everything else (prefill, host slot mappings) takes the distinct blocks with
        the index of their rows, once per step."""
        cfg = self.config
        on_device = (ctx is not None and not ctx.is_prefill and isinstance(ctx.slot_mapping, Tensor)
                     and ctx.slot_mapping.device.type == "cuda")
        if on_device:
            if step is None or step.touched is None or layer_idx == 0:
                touched = torch.div(slots, cfg.block_size, rounding_mode="floor").to(torch.int32)
                if step is None:
                    return touched
                step.touched = touched
            return step.touched
        if step is None:
            return ops.touched_blocks(slots, cfg.block_size, cfg.num_blocks)
        if step.touched is None:
            step.touched = ops.touched_blocks(slots, cfg.block_size, cfg.num_blocks)
        return step.touched

    def _store_kv(self, k: Tensor, v: Tensor, layer_idx: int, slot_mapping: Tuple[int, ...],
                  _step: Optional[_StepTensors] = None, _ctx: Optional[InferenceContext] = None) -> None:
        """``cache[layer, slot] = row`` for every non-negative slot (flex_backend.py:116-142)."""
        cfg = self.config
        k_flat = k.reshape(-1, cfg.num_kv_heads, cfg.head_dim)
        v_flat = v.reshape(-1, cfg.num_kv_heads, cfg.head_dim)
        n = len(slot_mapping)
        if n != k_flat.shape[0]:
            # the reference fails in its boolean-mask indexing with this error type
            raise IndexError(
                f"The shape of the mask [{n}] at index 0 does not match the shape of the indexed tensor "
                f"{list(k_flat.shape)} at index 0"
            )
        if self._fp8:
            if k_flat.dtype not in (torch.float32, torch.bfloat16, torch.float16) or v_flat.dtype != k_flat.dtype:
                raise RuntimeError("an fp8 pool takes fp32, bf16 or fp16 rows (k and v of the same type)")
        elif k_flat.dtype != self.k_cache.dtype or v_flat.dtype != self.v_cache.dtype:
            raise RuntimeError("Index put requires the source and destination dtypes match")
        if n == 0:
            return
        slots = self._device_slots(slot_mapping, n, _step, k_flat, v_flat)
        k_flat, v_flat = k_flat.contiguous(), v_flat.contiguous()
        kc, vc = self._layer(layer_idx)
        if self._fp8:
            # rows are encoded with the tile's scale; a row that raises a tile's absmax re-rounds the tile
            touched = self._touched(_step, slots, _ctx, layer_idx)
            ops.kv_append_e4m3(kc, vc, self.k_scale[layer_idx], self.v_scale[layer_idx], k_flat, v_flat, slots,
                               cfg.block_size, touched)
            return
        ops.kv_scatter(kc, vc, k_flat, v_flat, slots)

    # ------------------------------------------------------------------ gather
    def _gather_kv_from_cache(self, layer_idx: int, block_tables, seq_lens) -> Tuple[Tensor, Tensor]:
        """Zero-padded ``[num_seqs, max(seq_lens), Hkv, D]`` copies (flex_backend.py:233-279)."""
        cfg = self.config
        num_seqs, max_len = len(block_tables), max(seq_lens)
        self._require_device(self.k_cache)
        tables = self._to_device(_padded_tables(block_tables))
        lens = self._to_device(np.asarray(seq_lens, dtype=np.int32)[:num_seqs])
        kc, vc = self._layer(layer_idx)
        return ops.kv_gather(kc, vc, tables, lens, max_len, cfg.block_size)

    # ------------------------------------------------------------------ decode
    def _decode_attention(self, q: Tensor, layer_idx: int, ctx: InferenceContext) -> Tensor:
        """One query token per sequence over its cached keys (flex_backend.py:187-231)."""
        batch, seq_len, num_heads, head_dim = q.shape
        assert seq_len == 1, "Decode should have seq_len=1"
        if ctx.block_tables is None or ctx.seq_lens is None:
            raise ValueError("Decode requires block_tables and seq_lens in context")
        mod = self._mask_predicate(ctx.block_mask)
        if mod is not None:
            return self._decode_masked(q, layer_idx, ctx, mod)
        window = self._mask_window(ctx.block_mask, self._window if self.window_in_decode else 0)
        if isinstance(ctx.block_mask, PagedMask) and ctx.block_mask.boundaries is not None:
            raise NotImplementedError("a document mask describes packed prefill rows, not a decode step")
        if window and self.pad_zero_keys:
            raise ValueError("pad_zero_keys cannot be combined with a sliding window in decode")
        cfg = self.config
        self._require_device(q, self.k_cache)
        step = self._step(ctx)
        if step.seq_lens is None:
            self._tables(step, ctx.block_tables[:batch])
            if isinstance(ctx.seq_lens, Tensor) and ctx.seq_lens.device.type == "cuda":
                # already on the device: used as it is, with no host copy (a caller replaying a captured graph
                # updates the tensor in place between replays, so a converted copy would go stale)
                if ctx.seq_lens.dtype != torch.int32 or not ctx.seq_lens.is_contiguous():
                    raise TypeError("a device-resident seq_lens must be a contiguous int32 tensor")
                step.seq_lens = ctx.seq_lens[:batch]
                if self.pad_zero_keys and batch > 0:
                    step.extra_zero = torch.zeros(batch, dtype=torch.int32, device=step.seq_lens.device)
            else:
                lens = self._lens(ctx.seq_lens, batch)
                step.seq_lens = self._to_device(lens.astype(np.int32))
                if self.pad_zero_keys and batch > 0:
                    step.extra_zero = self._to_device((lens.max() - lens).astype(np.int32))
        if (self.pad_zero_keys and batch > 0 and layer_idx == 0 and isinstance(ctx.seq_lens, Tensor)
                and ctx.seq_lens.device.type == "cuda"):
            # Lengths that live on the device may have been rewritten since the last pass (a caller replaying a
            # captured graph does exactly that), so the padding counts are recomputed from them at the first
            # layer of every pass, into the buffer every layer reads: a capture records these two operations.
            torch.sub(step.seq_lens.max(), step.seq_lens, out=step.extra_zero)
        q3 = q.contiguous().view(batch, num_heads, head_dim)
        ws = self._workspace_for(
            ops.decode_workspace_bytes(batch, num_heads, cfg.num_kv_heads, head_dim, self.k_cache.dtype))
        kc, vc = self._layer(layer_idx)
        ksc = self.k_scale[layer_idx] if self._fp8 else None
        vsc = self.v_scale[layer_idx] if self._fp8 else None
        out = ops.decode(q3, kc, vc, step.tables, step.seq_lens, cfg.block_size, self.scale, ws, step.extra_zero,
                         ksc, vsc, window=window)
        return out.view(batch, 1, num_heads, head_dim)

    def _decode_masked(self, q: Tensor, layer_idx: int, ctx: InferenceContext, mod) -> Tensor:
        """Decode under an arbitrary predicate, literally as the reference evaluates it (flex_backend.py:203-225):
        the one query row has q_idx 0, kv_idx runs over the batch's longest sequence, and the positions past a
        shorter sequence's end are zero rows that take part wherever the predicate keeps them."""
        cfg = self.config
        batch, _, num_heads, head_dim = q.shape
        self._require_device(q, self.k_cache)
        step = self._step(ctx)
        if step.ctx_lens is None:
            lens = self._lens(ctx.seq_lens, batch)
            self._tables(step, ctx.block_tables[:batch])
            step.ctx_lens = self._to_device(lens.astype(np.int32))
            step.q_lens = torch.ones(batch, dtype=torch.int32, device=q.device)
            step.q_starts = torch.arange(batch, dtype=torch.int32, device=q.device)
            step.max_q_len = int(lens.max()) if batch else 0  # (here: the key count of the mask)
        words = self._mask_bits(step, mod, batch, num_heads, torch.zeros((batch, 1), dtype=torch.int64), step.max_q_len)
        kc, vc = self._layer(layer_idx)
        out = ops.attend_masked(q.contiguous().view(batch, num_heads, head_dim), kc, vc, step.tables, step.ctx_lens,
                                step.q_lens, step.q_starts, 1, cfg.block_size, self.scale, words, step.mask_keys,
                                k_scale=self.k_scale[layer_idx] if self._fp8 else None,
                                v_scale=self.v_scale[layer_idx] if self._fp8 else None)
        return out.view(batch, 1, num_heads, head_dim)

    # ------------------------------------------------------------------ prefill
    def _prefill_attention(self, q: Tensor, k: Tensor, v: Tensor, ctx: InferenceContext) -> Tensor:
        """Causal attention over the step's own K/V, cache not read (flex_backend.py:144-185).

        The dense ``[B, T, Hkv, D]`` inputs are handed to the paged kernel as a
        pool of ``B`` blocks of ``T`` tokens with the identity block table.
        """
        mod = self._mask_predicate(ctx.block_mask)
        window = 0 if mod is not None else self._mask_window(ctx.block_mask, self._window)
        batch, seq_len, num_heads, head_dim = q.shape
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        if out.numel() == 0:
            return out
        dev = self._require_device(q, k, v)
        if mod is not None:
            # an arbitrary predicate over the step's own K/V (flex_backend.py:170-178): q_idx = kv_idx = position
            # in the step; the dense K/V are a pool of `batch` blocks of `seq_len` tokens, as below
            pos = torch.arange(seq_len, dtype=torch.int64)[None].expand(batch, seq_len)
            words = self._mask_bits(self._step(ctx), mod, batch, num_heads, pos, seq_len)
            ar = torch.arange(batch, dtype=torch.int32, device=dev)
            lens = torch.full((batch,), seq_len, dtype=torch.int32, device=dev)
            num_kv = k.shape[2]
            ops.attend_masked(q.contiguous().view(batch * seq_len, num_heads, head_dim),
                              k.contiguous().view(batch * seq_len, num_kv, head_dim),
                              v.contiguous().view(batch * seq_len, num_kv, head_dim),
                              ar.reshape(batch, 1).contiguous(), lens, lens, ar * seq_len, seq_len, seq_len, self.scale,
                              words, seq_len, out=out.view(batch * seq_len, num_heads, head_dim))
            return out
        first = self._mask_first_keys(ctx.block_mask, self._step(ctx), batch, seq_len, None)
        num_kv = k.shape[2]
        if num_heads != num_kv * self.num_heads_per_kv:
            raise RuntimeError(
                f"q has {num_heads} heads but k/v have {num_kv} x num_heads_per_kv={self.num_heads_per_kv}")
        ar = torch.arange(batch, dtype=torch.int32, device=dev)
        lens = torch.full((batch,), seq_len, dtype=torch.int32, device=dev)
        ops.prefill_paged(
            q.contiguous().view(batch * seq_len, num_heads, head_dim),
            k.contiguous().view(batch * seq_len, num_kv, head_dim),
            v.contiguous().view(batch * seq_len, num_kv, head_dim),
            ar.reshape(batch, 1).contiguous(), lens, lens, ar * seq_len, seq_len, seq_len, self.scale,
            out=out.view(batch * seq_len, num_heads, head_dim), window=window, row_first_key=first)
        return out

    def _prefill_paged(self, q: Tensor, layer_idx: int, ctx: InferenceContext) -> Tensor:
        """Chunked prefill: ``q[b]`` holds the last ``T`` positions of a context of ``seq_lens[b]`` keys."""
        mod = self._mask_predicate(ctx.block_mask)
        window = 0 if mod is not None else self._mask_window(ctx.block_mask, self._window)
        if ctx.block_tables is None or ctx.seq_lens is None:
            raise ValueError("Chunked prefill requires block_tables and seq_lens in context")
        cfg = self.config
        batch, seq_len, num_heads, head_dim = q.shape
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        if out.numel() == 0:
            return out
        self._require_device(q, self.k_cache)
        step = self._step(ctx)
        if step.ctx_lens is None:
            totals = self._lens(ctx.seq_lens, batch)
            chunk = totals - self._lens(ctx.prefix_lens, batch)
            if (chunk < 0).any() or (chunk > seq_len).any():
                raise ValueError("prefix_lens / seq_lens do not describe chunks of at most q.shape[1] tokens")
            self._tables(step, ctx.block_tables[:batch])
            step.ctx_lens = self._to_device(totals.astype(np.int32))
            step.q_lens = self._to_device(chunk.astype(np.int32))
            step.q_starts = self._to_device((np.arange(batch, dtype=np.int64) * seq_len).astype(np.int32))
            step.max_q_len = int(chunk.max()) if batch else 0
        first = None
        if isinstance(ctx.block_mask, PagedMask) and ctx.block_mask.boundaries is not None:
            first = self._mask_first_keys(ctx.block_mask, step, batch, seq_len, self._lens(ctx.prefix_lens, batch))
        out.zero_()  # rows past a sequence's chunk length are padding and stay zero
        kc, vc = self._layer(layer_idx)
        tables = step.tables
        if mod is not None:
            # an arbitrary predicate over the cached context: row t of sequence b has q_idx = prefix + t
            totals = self._lens(ctx.seq_lens, batch)
            pos = torch.from_numpy(self._lens(ctx.prefix_lens, batch)[:, None] + np.arange(seq_len, dtype=np.int64)[None, :])
            words = self._mask_bits(step, mod, batch, num_heads, pos, int(totals.max()))
            ops.attend_masked(q.contiguous().view(batch * seq_len, num_heads, head_dim), kc, vc, tables, step.ctx_lens,
                              step.q_lens, step.q_starts, step.max_q_len, cfg.block_size, self.scale, words,
                              step.mask_keys, out=out.view(batch * seq_len, num_heads, head_dim),
                              k_scale=self.k_scale[layer_idx] if self._fp8 else None,
                              v_scale=self.v_scale[layer_idx] if self._fp8 else None)
            return out
        if self._fp8:
            # The matrix-core kernel reads 16-bit pools: dequantise the blocks the tables name into a compact
            # pool (each block once, however many sequences share it) and renumber the tables to match.
            if q.dtype not in (torch.bfloat16, torch.float16):
                raise RuntimeError("prefill over an fp8 pool takes bf16 or fp16 queries")
            if step.fp8_blocks is None:
                uniq, inverse = torch.unique(step.tables.reshape(-1), return_inverse=True)
                step.fp8_blocks = uniq.to(torch.int32)
                step.fp8_tables = torch.where(step.tables.reshape(-1) < 0, -1, inverse).to(torch.int32).view(
                    step.tables.shape).contiguous()
            kc = ops.dequantize_blocks_e4m3(kc, self.k_scale[layer_idx], step.fp8_blocks, cfg.block_size, q.dtype)
            vc = ops.dequantize_blocks_e4m3(vc, self.v_scale[layer_idx], step.fp8_blocks, cfg.block_size, q.dtype)
            tables = step.fp8_tables
        q3 = q.contiguous().view(batch * seq_len, num_heads, head_dim)
        # a step of few rows over a long context: with a workspace the kernel spreads its keys over the device
        need = ops.prefill_workspace_bytes(q3, tables, step.max_q_len, cfg.block_size, cfg.num_kv_heads, window)
        ops.prefill_paged(q3, kc, vc, tables, step.ctx_lens, step.q_lens, step.q_starts, step.max_q_len,
                          cfg.block_size, self.scale, out=out.view(batch * seq_len, num_heads, head_dim), window=window,
                          row_first_key=first, workspace=self._workspace_for(need) if need else None)
        return out

    # ------------------------------------------------------------------ fp8 pool
    def quantize_from(self, k_pool: Tensor, v_pool: Tensor, layer_idx: int) -> None:
        """Fill one layer of an fp8 pool from full-precision pools of the same shape.

        ``k_pool`` / ``v_pool``: ``[total_slots, Hkv, D]`` in fp32, bf16 or fp16.
        Each (block, kv head) tile gets scale = absmax/448 and is stored as
        e4m3fn(x / scale).
        """
        if not self._fp8:
            raise RuntimeError("quantize_from() needs CacheConfig(kv_format='fp8_e4m3')")
        cfg = self.config
        self._require_device(k_pool, v_pool, self.k_cache)
        for src, dst, scale in ((k_pool, self.k_cache, self.k_scale), (v_pool, self.v_cache, self.v_scale)):
            if tuple(src.shape) != cfg.cache_shape[1:]:
                raise ValueError(f"pool of shape {tuple(src.shape)}, expected {cfg.cache_shape[1:]}")
            bits, sc = ops.quantize_kv_e4m3(src.contiguous(), cfg.block_size)
            dst[layer_idx].copy_(bits)
            scale[layer_idx].copy_(sc)


# name under which code written for the reference finds its backend
class FlexAttentionBackend(HipPagedAttentionBackend):
    """The reference's class name with the reference's numerics as defaults: a ragged decode batch attends
    the zero-padded keys the reference's unmasked SDPA sees (flex_backend.py:253-264, :227-229;
    ``pad_zero_keys=True``) and a configured sliding window is not applied in decode unless the context carries
    a mask (:220-225; ``window_in_decode=False``).  ``HipPagedAttentionBackend`` itself defaults to
    exact-length, windowed decode."""

    def __init__(self, config: CacheConfig, pad_zero_keys: bool = True, window_in_decode: bool = False) -> None:
        super().__init__(config, pad_zero_keys=pad_zero_keys, window_in_decode=window_in_decode)
