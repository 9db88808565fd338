"""Tensor-level wrappers of the C ABI (one function per ``pa_*`` entry point).

Each wrapper takes torch tensors that already live on the HIP device, passes
their raw pointers, sizes and the current stream to ``libpaged_attn.so`` and
raises ``PagedAttnError`` on a negative status.  No computation happens in
Python and nothing is routed to torch kernels.
"""

from __future__ import annotations

from typing import NamedTuple, Optional, Tuple

import torch
from torch import Tensor

from . import _lib

PA_DTYPE = {torch.float32: _lib.PA_F32, torch.bfloat16: _lib.PA_BF16, torch.float16: _lib.PA_F16,
            torch.float8_e4m3fn: _lib.PA_FP8_E4M3, torch.uint8: _lib.PA_FP8_E4M3}


def _ptr(t: Optional[Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream(t: Tensor) -> Optional[int]:
    if t.device.type != "cuda":
        raise RuntimeError(f"libpaged_attn computes only on a HIP device; got a tensor on {t.device}")
    return torch.cuda.current_stream(t.device).cuda_stream or None


def _run(name: str, *args) -> None:
    _lib.check(name, getattr(_lib.load(), name)(*args))


def kv_scatter(k_cache: Tensor, v_cache: Tensor, k_src: Tensor, v_src: Tensor, slots: Tensor) -> None:
    """``cache[slots[i]] = src[i]``; caches ``[total_slots, Hkv, D]``, src ``[N, Hkv, D]``, slots int64 ``[N]``."""
    total_slots, hkv, d = k_cache.shape
    _run("pa_kv_scatter", _ptr(k_cache), _ptr(v_cache), _ptr(k_src), _ptr(v_src), _ptr(slots), slots.numel(),
         total_slots, hkv, d, k_cache.element_size(), _stream(k_cache))


def kv_gather(k_cache: Tensor, v_cache: Tensor, block_tables: Tensor, seq_lens: Tensor, max_len: int,
              block_size: int, out: Optional[Tuple[Tensor, Tensor]] = None) -> Tuple[Tensor, Tensor]:
    """Zero-padded ``[B, max_len, Hkv, D]`` copies; block_tables int32 ``[B, W]`` (-1 padded), seq_lens int32.
    ``out``: a pair of contiguous tensors of that shape and the pool's type to write into."""
    total_slots, hkv, d = k_cache.shape
    batch = block_tables.shape[0]
    if out is None:
        k_out = torch.empty((batch, max_len, hkv, d), dtype=k_cache.dtype, device=k_cache.device)
        v_out = torch.empty_like(k_out)
    else:
        k_out, v_out = out
        for t in (k_out, v_out):
            if tuple(t.shape) != (batch, max_len, hkv, d) or t.dtype != k_cache.dtype or not t.is_contiguous():
                raise ValueError("kv_gather: out tensors must be contiguous [B, max_len, Hkv, D] of the pool's type")
    _run("pa_kv_gather", _ptr(k_cache), _ptr(v_cache), _ptr(k_out), _ptr(v_out), _ptr(block_tables),
         block_tables.shape[1], _ptr(seq_lens), batch, max_len, total_slots // block_size, block_size, hkv, d,
         k_cache.element_size(), _stream(k_cache))
    return k_out, v_out


def decode_workspace_bytes(batch: int, num_q_heads: int, num_kv_heads: int, head_dim: int,
                           kv_dtype: torch.dtype) -> int:
    """Bytes of workspace ``decode`` needs for these shapes (independent of the sequence lengths)."""
    n = int(_lib.load().pa_decode_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, PA_DTYPE[kv_dtype]))
    if n == 0:
        raise _lib.PagedAttnError("pa_decode_workspace_bytes", 0, _lib.last_error())
    return n


def decode_workspace(q: Tensor, k_cache: Tensor) -> Tensor:
    """A fresh workspace tensor sized for ``decode(q, k_cache, ...)``, zero-filled: the library's arrival
    counters at its start must read zero before the first call that uses them."""
    batch, hq, d = q.shape
    n = decode_workspace_bytes(batch, hq, k_cache.shape[1], d, k_cache.dtype)
    return torch.zeros(n, dtype=torch.uint8, device=q.device)


def decode(q: Tensor, k_cache: Tensor, v_cache: Tensor, block_tables: Tensor, seq_lens: Tensor, block_size: int,
           scale: float, workspace: Tensor, extra_zero_keys: Optional[Tensor] = None,
           k_scale: Optional[Tensor] = None, v_scale: Optional[Tensor] = None, out: Optional[Tensor] = None,
           entry: str = "pa_decode", window: int = 0) -> Tensor:
    """Paged decode attention; q ``[B, Hq, D]`` -> out ``[B, Hq, D]`` (same dtype).

    ``entry`` may name ``pa_decode_split`` or ``pa_decode_reduce`` to run one pass only; ``window`` > 0
    restricts every sequence to its last ``window`` keys.
    """
    batch, hq, d = q.shape
    total_slots, hkv, _ = k_cache.shape
    if out is None:
        out = torch.empty_like(q)
    _run(entry, _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(block_tables), block_tables.shape[1],
         _ptr(seq_lens), _ptr(extra_zero_keys), _ptr(k_scale), _ptr(v_scale), batch, hq, hkv, d, block_size,
         total_slots // block_size, float(scale), int(window), PA_DTYPE[q.dtype], PA_DTYPE[k_cache.dtype],
         _ptr(workspace),
         workspace.numel() * workspace.element_size(), _stream(q))
    return out


def decode_static(q: Tensor, k_cache: Tensor, v_cache: Tensor, block_tables: Tensor, seq_lens: Tensor,
                  block_size: int, scale: float, extra_zero_keys: Optional[Tensor] = None,
                  k_scale: Optional[Tensor] = None, v_scale: Optional[Tensor] = None, out: Optional[Tensor] = None,
                  window: int = 0) -> Tensor:
    """``decode`` through ``pa_decode_static``: the partials go to the library's own fixed scratch array, the
    call allocates nothing (pass ``out``); shapes beyond the scratch raise ``PagedAttnError``."""
    batch, hq, d = q.shape
    total_slots, hkv, _ = k_cache.shape
    if out is None:
        out = torch.empty_like(q)
    _run("pa_decode_static", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(block_tables),
         block_tables.shape[1], _ptr(seq_lens), _ptr(extra_zero_keys), _ptr(k_scale), _ptr(v_scale), batch, hq, hkv,
         d, block_size, total_slots // block_size, float(scale), int(window), PA_DTYPE[q.dtype],
         PA_DTYPE[k_cache.dtype], _stream(q))
    return out


def prefill_workspace_bytes(q: Tensor, block_tables: Tensor, max_q_len: int, block_size: int, num_kv_heads: int,
                            window: int = 0) -> int:
    """Bytes of workspace with which ``prefill_paged`` spreads a launch of few rows over the device (0: the launch
    fills it anyway, or its shapes have no split kernel)."""
    total_q, hq, d = q.shape
    if q.dtype not in PA_DTYPE:
        return 0
    return int(_lib.load().pa_prefill_workspace_bytes(block_tables.shape[0], int(max_q_len), total_q,
                                                      block_tables.shape[1], block_size, int(window), hq,
                                                      num_kv_heads, d, PA_DTYPE[q.dtype]))


def prefill_paged(q: Tensor, k_cache: Tensor, v_cache: Tensor, block_tables: Tensor, ctx_lens: Tensor,
                  q_lens: Tensor, q_starts: Tensor, max_q_len: int, block_size: int, scale: float,
                  out: Optional[Tensor] = None, window: int = 0, row_first_key: Optional[Tensor] = None,
                  rowwise: bool = False, workspace: Optional[Tensor] = None) -> Tensor:
    """Causal prefill over a paged context; q ``[total_q, Hq, D]`` packed rows; ``window`` > 0 adds the
    sliding window (a row at position p sees keys p - window < j <= p); ``row_first_key`` (int32 per q row,
    non-decreasing along a sequence) adds a per-row first key, e.g. the start of the row's document;
    ``rowwise`` selects the vector kernel (``pa_prefill_paged_rowwise``) also where a matrix-core kernel exists;
    ``workspace`` (uint8, ``prefill_workspace_bytes`` or more) lets a launch of few rows split its keys over
    several workgroups (``pa_prefill_paged_ws``)."""
    total_q, hq, d = q.shape
    if row_first_key is not None and (row_first_key.dtype != torch.int32 or row_first_key.numel() != total_q):
        raise ValueError("row_first_key must hold one int32 per q row")
    total_slots, hkv, _ = k_cache.shape
    if out is None:
        out = torch.empty_like(q)
    args = (_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(block_tables), block_tables.shape[1],
            _ptr(ctx_lens), _ptr(q_lens), _ptr(q_starts), _ptr(row_first_key) if row_first_key is not None else None,
            block_tables.shape[0], max_q_len, hq, hkv, d, block_size, total_slots // block_size, float(scale),
            int(window), PA_DTYPE[q.dtype], _stream(q))
    if workspace is not None and not rowwise:
        # (``pa_prefill_paged_ws``: the launch is cut into pieces over the keys when it has too few rows for the device)
        _run("pa_prefill_paged_ws", *args, total_q, _ptr(workspace), workspace.numel() * workspace.element_size())
    else:
        _run("pa_prefill_paged_rowwise" if rowwise else "pa_prefill_paged", *args)
    return out


def pack_mask(keep: Tensor) -> Tensor:
    """Bits of a boolean mask ``[rows, heads (or 1), keys]`` as int32 words ``[rows, heads, ceil(keys / 32)]``
    (bit j of word j // 32 = keep[..., j]), the layout ``attend_masked`` takes.  Packed with byte arithmetic, a
    bounded number of rows at a time: the temporaries stay near the size of the boolean input."""
    rows, heads, keys = keep.shape
    words = max(1, -(-keys // 32))
    out = torch.empty((rows, heads, words), dtype=torch.int32, device=keep.device)
    per_row = max(1, heads * words * 32)
    chunk = max(1, (1 << 27) // per_row)  # about 128 MiB of bytes per round
    for at in range(0, rows, chunk):
        part = keep[at: at + chunk]
        n = part.shape[0]
        if keys == words * 32:
            bits = part.contiguous().view(torch.uint8) if part.dtype == torch.bool else part.to(torch.uint8)
        else:
            bits = torch.zeros((n, heads, words * 32), dtype=torch.uint8, device=keep.device)
            bits[..., :keys] = part
        bits = bits.reshape(n, heads, words * 4, 8)
        byte = bits[..., 0].clone()
        for k in range(1, 8):
            byte |= bits[..., k] << k
        out[at: at + n] = byte.contiguous().view(torch.int32).view(n, heads, words)  # little-endian: byte 0 = bits 0..7
    return out


def attend_masked(q: Tensor, k_cache: Tensor, v_cache: Tensor, block_tables: Tensor, ctx_lens: Tensor, q_lens: Tensor,
                  q_starts: Tensor, max_q_len: int, block_size: int, scale: float, mask_words: Tensor, n_keys: int,
                  out: Optional[Tensor] = None, k_scale: Optional[Tensor] = None,
                  v_scale: Optional[Tensor] = None) -> Tensor:
    """Attention of packed q rows ``[total_q, Hq, D]`` over a paged context under an arbitrary mask
    (``pa_attend_masked``): ``mask_words`` int32 ``[total_q, 1 or Hq, words]`` from ``pack_mask``; row r attends
    key j < n_keys iff its bit is set; keys at or past ``ctx_lens[b]`` are zero rows.  An fp8-e4m3 pool comes with
    its ``k_scale`` / ``v_scale``."""
    total_q, hq, d = q.shape
    total_slots, hkv, _ = k_cache.shape
    if mask_words.dtype != torch.int32 or mask_words.dim() != 3 or mask_words.shape[0] != total_q:
        raise ValueError("mask_words must be int32 [total_q, heads, words]")
    if out is None:
        out = torch.empty_like(q)
    _run("pa_attend_masked", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(block_tables),
         block_tables.shape[1], _ptr(ctx_lens), _ptr(q_lens), _ptr(q_starts), _ptr(mask_words), mask_words.shape[1],
         mask_words.shape[2], int(n_keys), block_tables.shape[0], max_q_len, hq, hkv, d, block_size,
         total_slots // block_size, float(scale), PA_DTYPE[q.dtype], PA_DTYPE[k_cache.dtype], _ptr(k_scale),
         _ptr(v_scale), _stream(q))
    return out


def quantize_kv_e4m3(pool: Tensor, block_size: int) -> Tuple[Tensor, Tensor]:
    """e4m3fn bytes (as ``torch.float8_e4m3fn``) and ``float32 [num_blocks, Hkv]`` scales of a pool."""
    total_slots, hkv, d = pool.shape
    num_blocks = total_slots // block_size
    dst = torch.empty(pool.shape, dtype=torch.float8_e4m3fn, device=pool.device)
    scale = torch.empty((num_blocks, hkv), dtype=torch.float32, device=pool.device)
    _run("pa_quantize_kv_e4m3", _ptr(pool), _ptr(dst), _ptr(scale), num_blocks, block_size, hkv, d,
         PA_DTYPE[pool.dtype], _stream(pool))
    return dst, scale


class TouchedBlocks(NamedTuple):
    """The distinct blocks a slot list writes to and the index of its rows by block that ``pa_kv_append_e4m3``
    takes: rows ``row_order[block_start[i]:block_start[i + 1]]`` are the tokens whose slots fall in ``blocks[i]``."""

    blocks: Tensor       # int32 [n_touched]
    row_order: Tensor    # int32 [n_rows], token indices grouped by block
    block_start: Tensor  # int32 [n_touched + 1]


def touched_blocks(slots: Tensor, block_size: int, num_blocks: int) -> TouchedBlocks:
    """Distinct blocks (int32, on the device) that the non-negative, in-pool slots fall in, with the rows of
    each: an append workgroup then reads the slots of its own block instead of the whole list."""
    blocks = torch.div(slots, block_size, rounding_mode="floor")
    rows = torch.nonzero((slots >= 0) & (blocks < num_blocks)).reshape(-1)
    uniq, inverse, counts = torch.unique(blocks[rows], return_inverse=True, return_counts=True)
    order = rows[torch.argsort(inverse, stable=True)]
    start = torch.zeros(uniq.numel() + 1, dtype=torch.int32, device=slots.device)
    start[1:] = torch.cumsum(counts, 0)
    return TouchedBlocks(uniq.to(torch.int32), order.to(torch.int32).contiguous(), start)


def _touched_args(touched, slots: Tensor, block_size: int, num_blocks: int):
    """(blocks, row_order, block_start) for the append calls: ``touched`` is a TouchedBlocks, a bare int32 tensor
    of blocks (no index: every workgroup scans the slot list) or None (computed here)."""
    if touched is None:
        touched = touched_blocks(slots, block_size, num_blocks)
    if isinstance(touched, TouchedBlocks):
        return touched.blocks, touched.row_order, touched.block_start
    return touched, None, None


def kv_append_e4m3(k_cache: Tensor, v_cache: Tensor, k_scale: Tensor, v_scale: Tensor, k_src: Tensor, v_src: Tensor,
                   slots: Tensor, block_size: int, touched=None) -> None:
    """Append rows to an fp8-e4m3 pool with the "re-round on growth" policy of ``pa_kv_append_e4m3``.

    k_cache/v_cache ``[total_slots, Hkv, D]`` float8_e4m3fn, scales ``float32 [num_blocks, Hkv]`` (updated in
    place), k_src/v_src ``[N, Hkv, D]`` fp32/bf16/fp16, slots ``int64 [N]``.  ``touched`` (a ``TouchedBlocks``
    from ``touched_blocks``, or a bare int32 tensor of the distinct target blocks without the row index) is
    computed with torch when not given.
    """
    total_slots, hkv, d = k_cache.shape
    num_blocks = total_slots // block_size
    blocks, order, start = _touched_args(touched, slots, block_size, num_blocks)
    _run("pa_kv_append_e4m3", _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale), _ptr(k_src), _ptr(v_src),
         _ptr(slots), slots.numel(), _ptr(blocks), blocks.numel(), _ptr(order), _ptr(start), num_blocks, block_size,
         hkv, d, PA_DTYPE[k_src.dtype], _stream(k_cache))


def rope_kv_append(q: Tensor, k_src: Tensor, v_src: Tensor, cos: Tensor, sin: Tensor, k_cache: Optional[Tensor],
                   v_cache: Optional[Tensor], slots: Optional[Tensor], positions: Optional[Tensor] = None,
                   q_out: Optional[Tensor] = None, k_out: Optional[Tensor] = None) -> Tensor:
    """Rotary embedding of q and k fused with the KV append (``pa_rope_kv_append``).

    q ``[N, Hq, D]``, k_src/v_src ``[N, Hkv, D]``, cos/sin ``[R, D]`` of the same dtype; ``positions`` int32 ``[N]``
    picks the table row per token (None: row i for token i).  The rotated k and v go to the caches at ``slots``
    (int64 ``[N]``; None: no cache write) and the rotated k also to ``k_out`` when given.  Returns rotated q
    (``q_out``, or q itself rotated in place when ``q_out`` is None).
    """
    n, hq, d = q.shape
    hkv = k_src.shape[1]
    if q_out is None:
        q_out = q
    for t in (k_src, v_src, cos, sin):
        if t.dtype != q.dtype:
            raise RuntimeError("q, k, v, cos and sin must have the same dtype")
    if positions is not None and positions.dtype != torch.int32:
        raise ValueError("positions must be int32")
    if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != d:
        raise ValueError("cos / sin must be [rows, head_dim]")
    total_slots = k_cache.shape[0] if k_cache is not None else 0
    _run("pa_rope_kv_append", _ptr(q), _ptr(q_out), _ptr(k_src), _ptr(v_src), _ptr(k_out), _ptr(k_cache),
         _ptr(v_cache), _ptr(cos), _ptr(sin), _ptr(positions), cos.shape[0], _ptr(slots), n, total_slots, hq, hkv, d,
         PA_DTYPE[q.dtype], _stream(q))
    return q_out


def rope_kv_append_e4m3(q: Tensor, k_src: Tensor, v_src: Tensor, cos: Tensor, sin: Tensor, k_cache: Tensor,
                        v_cache: Tensor, k_scale: Tensor, v_scale: Tensor, slots: Tensor, block_size: int,
                        positions: Optional[Tensor] = None, q_out: Optional[Tensor] = None,
                        touched=None) -> Tensor:
    """``rope_kv_append`` into an fp8-e4m3 pool (``pa_rope_kv_append_e4m3``): k is rotated while the fp8 append
    reads it; arguments as in ``rope_kv_append`` and ``kv_append_e4m3``."""
    n, hq, d = q.shape
    total_slots, hkv, _ = k_cache.shape
    num_blocks = total_slots // block_size
    if q_out is None:
        q_out = q
    for t in (k_src, v_src, cos, sin):
        if t.dtype != q.dtype:
            raise RuntimeError("q, k, v, cos and sin must have the same dtype")
    if positions is not None and positions.dtype != torch.int32:
        raise ValueError("positions must be int32")
    blocks, order, start = _touched_args(touched, slots, block_size, num_blocks)
    _run("pa_rope_kv_append_e4m3", _ptr(q), _ptr(q_out), _ptr(k_src), _ptr(v_src), _ptr(k_cache), _ptr(v_cache),
         _ptr(k_scale), _ptr(v_scale), _ptr(cos), _ptr(sin), _ptr(positions), cos.shape[0], _ptr(slots), n,
         _ptr(blocks), blocks.numel(), _ptr(order), _ptr(start), num_blocks, block_size, hq, hkv, d,
         PA_DTYPE[q.dtype], _stream(q))
    return q_out


def dequantize_blocks_e4m3(cache: Tensor, scale: Tensor, block_ids: Tensor, block_size: int,
                           dtype: torch.dtype = torch.bfloat16) -> Tensor:
    """Compact 16-bit pool ``[len(block_ids) * block_size, Hkv, D]`` holding the listed blocks of an fp8-e4m3
    pool dequantised (``pa_dequantize_blocks_e4m3``); ``block_ids`` int32 on the device."""
    total_slots, hkv, d = cache.shape
    if block_ids.dtype != torch.int32:
        raise ValueError("block_ids must be int32")
    dst = torch.empty((block_ids.numel() * block_size, hkv, d), dtype=dtype, device=cache.device)
    _run("pa_dequantize_blocks_e4m3", _ptr(cache), _ptr(scale), _ptr(block_ids), block_ids.numel(), _ptr(dst),
         total_slots // block_size, block_size, hkv, d, PA_DTYPE[dtype], _stream(cache))
    return dst
