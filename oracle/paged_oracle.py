"""CPU restatement of the reference's paged attention path.  TEST INFRASTRUCTURE.

Nothing in the product imports this file: it exists so that tests, the smoke
check and the CPU-baseline leg of the benchmark can compare the HIP path with
an independent statement of what the reference computes.  It never imports
the reference; each function cites the reference lines it restates
(paths relative to rollouts/rollouts/inference/).

Two families:

* ``*_literal`` functions follow the reference statement by statement with the
  same PyTorch calls (Python gather loop, ``repeat_interleave``,
  ``scaled_dot_product_attention``).  They are the timed CPU baseline and the
  arbiter for the reference's ragged-batch zero-padding behaviour.
* the numpy functions compute the same mathematics directly in float64
  (explicit softmax) at exact sequence lengths; they are what the HIP results
  are compared with.

How each function is pinned (see tests/test_oracle.py):
  kv_scatter            the reference's own assertion (slots 0..3 -> rows 0..3,
                        examples/inference/test_kv_cache.py:106-111), closed form
  kv_gather_padded      closed form slot = bt[pos//bs]*bs + pos%bs, brute force
                        loop on small pools, gather(scatter(x)) = x
  paged_decode          pure-Python softmax on tiny inputs; torch SDPA on the
                        gathered tensors; invariance under pool permutation;
                        GQA vs explicitly expanded heads; constant V
  paged_decode(pad_zero_keys=True)
                        equals ``decode_literal`` (SDPA over the zero-padded
                        batch) and the closed form with (Lmax-L) extra e^(-m)
                        terms in the denominator
  dense_prefill         torch SDPA is_causal=True with the recipe and tolerance
                        of the reference's test (test_kv_cache.py:321-342)
  paged_prefill_chunk   rows [P:P+C] of dense_prefill over the whole sequence;
                        P=0 equals dense_prefill
  window= (decode, prefill)
                        torch SDPA with the explicit boolean mask
                        q_idx >= kv_idx and q_idx - kv_idx < window, the
                        recipe of the reference's debug_swa.py; window >= length
                        equals no window; decode equals the last prefill row
  doc_lens= (prefill)   torch SDPA with the explicit boolean mask evaluated by a
                        scalar restatement of document_mask's loop
                        (attention/mask.py:173-186) entry by entry; equals
                        independent causal attention on each document alone
  rope_tables           closed form angle = pos * theta**(-2i/D) in float64; cos^2 +
                        sin^2 = 1; both halves of a row equal; position 0 -> (1, 0)
  rope_literal          rope_exact (complex multiplication in float64) within the
                        rounding of the type; position 0 is the identity; norms of
                        (x_i, x_{i+D/2}) pairs kept; q.k after rotation depends only
                        on the distance between the two positions
  quantize_kv_e4m3      torch.float8_e4m3fn conversion (library definition of
                        OCP e4m3fn, round to nearest even), known values
                        464 -> 448, 2**-10 -> 0, max 448
  append_kv_e4m3        (a policy of this build, the reference has no fp8 pool)
                        appending a whole block in one call equals
                        quantize_kv_e4m3 of that block bit for bit; rows of
                        non-increasing magnitude leave earlier bytes and the
                        scale untouched; after any append order the dequantised
                        pool is within two e4m3 roundings of the input
Parity unpinned by any test of the reference itself: decode values, the
gather and ragged batches (the reference only asserts shapes there).
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

# --------------------------------------------------------------------------- helpers


def to_f64(x) -> np.ndarray:
    if isinstance(x, torch.Tensor):
        return x.detach().to(torch.float64).cpu().numpy()
    return np.asarray(x, dtype=np.float64)


def slot_of(blocks: Sequence[int], pos: int, block_size: int) -> int:
    """Slot of token position ``pos``; -1 if the table is too short (context.py:35-42, :78-85)."""
    idx = pos // block_size
    if idx >= len(blocks):
        return -1
    return int(blocks[idx]) * block_size + pos % block_size


# --------------------------------------------------------------------------- scatter / gather


def kv_scatter(k_cache, v_cache, k_src, v_src, slots: Sequence[int]) -> None:
    """In place: ``cache[s] = src[i]`` for every ``s = slots[i] >= 0`` (flex_backend.py:116-142).

    ``*_cache``: one layer ``[total_slots, Hkv, D]``; ``*_src``: ``[N, Hkv, D]``
    (numpy arrays or torch tensors; rows are copied, never converted).
    """
    slots = np.asarray(slots, dtype=np.int64)
    assert slots.shape[0] == k_src.shape[0] == v_src.shape[0]
    keep = np.nonzero(slots >= 0)[0]
    for i in keep:  # in order, so that on duplicate slots the last writer wins as on CPU
        k_cache[int(slots[i])] = k_src[int(i)]
        v_cache[int(slots[i])] = v_src[int(i)]


def kv_gather_padded(k_cache, v_cache, block_tables, seq_lens, block_size: int):
    """Zero-padded ``[B, max(seq_lens), Hkv, D]`` gather (flex_backend.py:233-279).

    Positions past a sequence's length, and positions whose block index is past
    the end of that sequence's table (:274), stay zero.  Works on numpy arrays
    or torch tensors and returns the same kind.
    """
    num_seqs, max_len = len(block_tables), int(max(seq_lens))
    shape = (num_seqs, max_len) + tuple(k_cache.shape[1:])
    if isinstance(k_cache, torch.Tensor):
        k_out = torch.zeros(shape, dtype=k_cache.dtype)
        v_out = torch.zeros(shape, dtype=v_cache.dtype)
    else:
        k_out = np.zeros(shape, dtype=k_cache.dtype)
        v_out = np.zeros(shape, dtype=v_cache.dtype)
    for b, (blocks, n) in enumerate(zip(block_tables, seq_lens)):
        blocks = np.asarray(blocks, dtype=np.int64)
        n_ok = min(int(n), len(blocks) * block_size)
        if n_ok <= 0:
            continue
        pos = np.arange(n_ok)
        slots = blocks[pos // block_size] * block_size + pos % block_size
        if isinstance(k_cache, torch.Tensor):
            idx = torch.from_numpy(slots)
            k_out[b, :n_ok] = k_cache[idx]
            v_out[b, :n_ok] = v_cache[idx]
        else:
            k_out[b, :n_ok] = k_cache[slots]
            v_out[b, :n_ok] = v_cache[slots]
    return k_out, v_out


def kv_gather_loop(k_cache, v_cache, block_tables, seq_lens, block_size: int):
    """The reference's two-level loop, token by token (flex_backend.py:266-277).  Small inputs only."""
    num_seqs, max_len = len(block_tables), int(max(seq_lens))
    shape = (num_seqs, max_len) + tuple(k_cache.shape[1:])
    k_out = torch.zeros(shape, dtype=k_cache.dtype)
    v_out = torch.zeros(shape, dtype=v_cache.dtype)
    for b, (blocks, n) in enumerate(zip(block_tables, seq_lens)):
        for pos in range(int(n)):
            slot = slot_of(blocks, pos, block_size)
            if slot >= 0:
                k_out[b, pos] = k_cache[slot]
                v_out[b, pos] = v_cache[slot]
    return k_out, v_out


# --------------------------------------------------------------------------- attention (float64, explicit)


def document_of(boundaries: Sequence[int], idx: np.ndarray) -> np.ndarray:
    """Document index of each position: the number of document ends at or before it
    (attention/mask.py:176-185: ``doc = i + 1`` for the last boundary with ``idx >= boundary``);
    positions past the last document therefore form one more document."""
    ends = np.asarray(list(boundaries)[1:], dtype=np.int64)
    return (np.asarray(idx)[..., None] >= ends).sum(axis=-1)


def document_boundaries(seq_lens: Sequence[int]) -> List[int]:
    """Running sums of the document lengths, starting at 0 (attention/mask.py:168-171)."""
    bounds = [0]
    for n in seq_lens:
        bounds.append(bounds[-1] + int(n))
    return bounds


def _attend_rows(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, n_zero: int = 0,
                 causal_offset: Optional[int] = None, window: int = 0,
                 boundaries: Optional[Sequence[int]] = None) -> np.ndarray:
    """softmax(scale * q k^T) v for one kv head group.

    q ``[R, n_rep, D]``, k/v ``[L, D]`` -> ``[R, n_rep, D]``.  ``n_zero`` extra
    all-zero keys (logit 0, value 0) join the softmax.  ``causal_offset``: row
    r sits at position ``causal_offset + r`` and may only see keys
    ``j <= causal_offset + r``; with ``window`` > 0 also only keys with
    ``position - j < window`` (attention/mask.py:83-89); with ``boundaries``
    (document starts and the final end) also only keys of the row's own
    document (attention/mask.py:173-186).
    """
    logits = scale * np.einsum("rhd,ld->rhl", q, k)  # [R, n_rep, L]
    if causal_offset is not None:
        rows = np.arange(q.shape[0])[:, None, None]
        cols = np.arange(k.shape[0])[None, None, :]
        seen = cols <= causal_offset + rows
        if window > 0:
            seen &= (causal_offset + rows) - cols < window
        if boundaries is not None:
            seen &= document_of(boundaries, causal_offset + rows) == document_of(boundaries, cols)
        logits = np.where(seen, logits, -np.inf)
    m = logits.max(axis=-1, keepdims=True) if logits.shape[-1] else np.full(logits.shape[:-1] + (1,), -np.inf)
    if n_zero > 0:
        m = np.maximum(m, 0.0)
    m = np.where(np.isfinite(m), m, 0.0)
    p = np.exp(logits - m)
    den = p.sum(axis=-1, keepdims=True) + n_zero * np.exp(-m)
    out = np.einsum("rhl,ld->rhd", p, v)
    with np.errstate(invalid="ignore", divide="ignore"):
        return np.where(den > 0, out / den, 0.0)


def paged_decode(q, k_cache, v_cache, block_tables, seq_lens, block_size: int, scale: float,
                 pad_zero_keys: bool = False, window: int = 0) -> np.ndarray:
    """Decode attention at exact lengths (flex_backend.py:187-231 with a length mask).

    q ``[B, Hq, D]``; caches ``[total_slots, Hkv, D]``; returns float64 ``[B, Hq, D]``.
    Query head h reads kv head ``h // (Hq/Hkv)`` - the mapping ``repeat_interleave``
    on dim 1 produces (:215-217).  Positions whose block is missing from the
    table are all-zero keys, as in the reference's gather (:274).  With
    ``pad_zero_keys`` every sequence additionally sees ``max(seq_lens) - len``
    zero keys: the reference's unmasked attention over the zero-padded batch.
    A sequence with no keys at all yields zeros.  ``window`` > 0: the query (at
    position len-1) sees only keys ``j`` with ``len-1 - j < window``
    (attention/mask.py:83-89 applied to the decode row).
    """
    q, kc, vc = to_f64(q), to_f64(k_cache), to_f64(v_cache)
    batch, hq, d = q.shape
    hkv = kc.shape[1]
    n_rep = hq // hkv
    max_len = int(max(seq_lens)) if len(seq_lens) else 0
    out = np.zeros((batch, hq, d))
    for b in range(batch):
        n = int(seq_lens[b])
        blocks = np.asarray(block_tables[b], dtype=np.int64)
        n_ok = max(0, min(n, len(blocks) * block_size))
        first = max(0, n - window) if window > 0 else 0
        pos = np.arange(min(first, n_ok), n_ok)
        slots = blocks[pos // block_size] * block_size + pos % block_size
        n_zero = (n - max(n_ok, first)) + (max_len - n if pad_zero_keys else 0)
        for g in range(hkv):
            qg = q[b, g * n_rep : (g + 1) * n_rep][None]  # [1, n_rep, D]
            out[b, g * n_rep : (g + 1) * n_rep] = _attend_rows(qg, kc[slots, g], vc[slots, g], scale, n_zero)[0]
    return out


def dense_prefill(q, k, v, scale: float, window: int = 0, doc_lens: Optional[Sequence[int]] = None) -> np.ndarray:
    """Causal attention over the step's own K/V (flex_backend.py:144-185, SDPA is_causal=True; with
    ``window`` the flex_attention path under causal_sliding_window_mask, attention/mask.py:56-100; with
    ``doc_lens`` under the packed-document mask of create_document_mask, attention/mask.py:141-191).

    q ``[B, T, Hq, D]``, k/v ``[B, T, Hkv, D]`` -> float64 ``[B, T, Hq, D]``.
    """
    q, k, v = to_f64(q), to_f64(k), to_f64(v)
    batch, t, hq, d = q.shape
    hkv = k.shape[2]
    n_rep = hq // hkv
    out = np.zeros_like(q)
    bounds = document_boundaries(doc_lens) if doc_lens is not None else None
    for b in range(batch):
        for g in range(hkv):
            sl = slice(g * n_rep, (g + 1) * n_rep)
            out[b, :, sl] = _attend_rows(q[b, :, sl], k[b, :, g], v[b, :, g], scale, causal_offset=0, window=window,
                                         boundaries=bounds)
    return out


def paged_prefill_chunk(q, k_cache, v_cache, block_tables, prefix_lens, chunk_lens, block_size: int,
                        scale: float, window: int = 0, doc_lens: Optional[Sequence[int]] = None) -> np.ndarray:
    """Chunked prefill over a cached prefix (composition; not a reference function).

    Defined as: gather keys ``0 .. P+C-1`` through the block table
    (flex_backend.py:233-279) and attend with a bottom-right aligned causal
    mask, i.e. chunk row i (absolute position P+i) sees keys ``j <= P+i``.
    The chunk's own K/V must already be in the cache.  q ``[B, Cmax, Hq, D]``;
    rows past ``chunk_lens[b]`` give zeros.  ``doc_lens``: documents packed
    into every sequence by absolute position (attention/mask.py:141-191).
    """
    q, kc, vc = to_f64(q), to_f64(k_cache), to_f64(v_cache)
    batch, cmax, hq, d = q.shape
    hkv = kc.shape[1]
    n_rep = hq // hkv
    out = np.zeros_like(q)
    bounds = document_boundaries(doc_lens) if doc_lens is not None else None
    for b in range(batch):
        p, c = int(prefix_lens[b]), int(chunk_lens[b])
        blocks = np.asarray(block_tables[b], dtype=np.int64)
        pos = np.arange(p + c)
        slots = blocks[pos // block_size] * block_size + pos % block_size
        for g in range(hkv):
            sl = slice(g * n_rep, (g + 1) * n_rep)
            out[b, :c, sl] = _attend_rows(q[b, :c, sl], kc[slots, g], vc[slots, g], scale, causal_offset=p,
                                          window=window, boundaries=bounds)
    return out


def paged_attend_masked(q, k_cache, v_cache, block_tables, ctx_lens, q_lens, keep, block_size: int,
                        scale: float) -> np.ndarray:
    """Attention under an arbitrary boolean mask: what the reference gets from ``flex_attention(q, k, v,
    block_mask=..., scale=...)`` (flex_backend.py:175-178 in prefill, :220-225 in decode) for the mask_mod the
    block mask was built from, stated densely.  q ``[B, Tmax, Hq, D]``; ``keep`` bool ``[B, Tmax, Hq or 1,
    n_keys]`` = mask_mod(b, h, q_idx, kv_idx) evaluated on every entry; keys are gathered through the block
    table with zero rows past ``ctx_lens[b]`` and for absent blocks (the zero-initialised gather of
    flex_backend.py:253-277); kv heads are repeated to the query heads (:213-216).  softmax over the kept keys
    only (a masked score is -inf); a row that keeps no key gives zeros, as flex_attention does; rows past
    ``q_lens[b]`` give zeros."""
    q, kc, vc = to_f64(q), to_f64(k_cache), to_f64(v_cache)
    keep = np.asarray(keep, dtype=bool)
    batch, tmax, hq, d = q.shape
    hkv = kc.shape[1]
    n_rep = hq // hkv
    n_keys = keep.shape[-1]
    num_blocks = kc.shape[0] // block_size
    out = np.zeros_like(q)
    for b in range(batch):
        blocks = np.asarray(block_tables[b], dtype=np.int64)
        k = np.zeros((n_keys, hkv, d))
        v = np.zeros((n_keys, hkv, d))
        for j in range(min(n_keys, int(ctx_lens[b]))):
            blk = j // block_size
            if blk < len(blocks) and 0 <= blocks[blk] < num_blocks:
                slot = blocks[blk] * block_size + j % block_size
                k[j], v[j] = kc[slot], vc[slot]
        for t in range(int(q_lens[b])):
            for h in range(hq):
                m = keep[b, t, h if keep.shape[2] > 1 else 0]
                if not m.any():
                    continue
                s = (k[m, h // n_rep] @ q[b, t, h]) * scale
                w = np.exp(s - s.max())
                out[b, t, h] = (w / w.sum()) @ v[m, h // n_rep]
    return out


# --------------------------------------------------------------------------- rotary embedding
# (rollouts/tools/functional_extractor/llama_functional.py; the step a model runs right before attention)


def rope_tables(positions: torch.Tensor, head_dim: int, theta: float = 10000.0,
                dtype: torch.dtype = torch.bfloat16) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos / sin tables, statement by statement (llama_functional.py:101-136): ``inv_freq[i] =
    theta**(-2i/D)`` in float32, angles = position * inv_freq, both halves of a row hold the same
    angles, cosine and sine taken in float32 and cast once.  positions ``[B, T]`` -> ``[B, T, D]`` each."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2).float() / head_dim))
    freqs = (inv_freq[None, :, None] @ positions[:, None, :].float()).transpose(1, 2)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rope_literal(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``(x * cos) + (rotate_half(x) * sin)`` with the same tensor operations, in the tensors' own type
    (llama_functional.py:68-72, :96-97).  x ``[N, H, D]``, cos/sin ``[N, D]`` (one row per token)."""
    half = x.shape[-1] // 2
    rotated = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return (x * cos[:, None, :]) + (rotated * sin[:, None, :])


def rope_exact(x, angles: np.ndarray) -> np.ndarray:
    """What the statement above computes, in float64 and in complex form: element i and element i + D/2 of a
    head are the real and imaginary part of a number that is multiplied by ``exp(1j * angle_i)``.
    x ``[N, H, D]``, angles ``[N, D/2]`` -> float64 ``[N, H, D]``."""
    x = to_f64(x)
    half = x.shape[-1] // 2
    z = (x[..., :half] + 1j * x[..., half:]) * np.exp(1j * np.asarray(angles, dtype=np.float64))[:, None, :]
    return np.concatenate([z.real, z.imag], axis=-1)


# --------------------------------------------------------------------------- literal restatement (torch)


def decode_literal(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables, seq_lens,
                   block_size: int, scale: float, vectorised_gather: bool = False) -> torch.Tensor:
    """The reference's decode, statement by statement (flex_backend.py:187-231, :233-279).

    q ``[B, 1, Hq, D]`` -> ``[B, 1, Hq, D]``.  Gathers a zero-padded batch with
    the token loop (or its vectorised equivalent), expands kv heads with
    ``repeat_interleave`` and calls SDPA without any mask.
    """
    gather = kv_gather_padded if vectorised_gather else kv_gather_loop
    k_g, v_g = gather(k_cache, v_cache, block_tables, seq_lens, block_size)
    n_rep = q.shape[2] // k_cache.shape[1]
    qt = q.transpose(1, 2)
    kt, vt = k_g.transpose(1, 2), v_g.transpose(1, 2)
    if n_rep > 1:
        kt = kt.repeat_interleave(n_rep, dim=1)
        vt = vt.repeat_interleave(n_rep, dim=1)
    out = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, is_causal=False, scale=scale)
    return out.transpose(1, 2)


def decode_per_sequence(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables, seq_lens,
                        block_size: int, scale: float) -> torch.Tensor:
    """Vectorised CPU restatement at exact lengths: per sequence index-gather + SDPA.

    The same library calls as the reference, minus the padding; this is the
    CPU baseline that stays runnable at the large configurations.
    """
    batch, _, hq, d = q.shape
    n_rep = hq // k_cache.shape[1]
    out = torch.empty_like(q)
    for b in range(batch):
        n = int(seq_lens[b])
        blocks = np.asarray(block_tables[b], dtype=np.int64)
        pos = np.arange(n)
        idx = torch.from_numpy(blocks[pos // block_size] * block_size + pos % block_size)
        kt = k_cache[idx].transpose(0, 1).unsqueeze(0)  # [1, Hkv, L, D]
        vt = v_cache[idx].transpose(0, 1).unsqueeze(0)
        if n_rep > 1:
            kt = kt.repeat_interleave(n_rep, dim=1)
            vt = vt.repeat_interleave(n_rep, dim=1)
        qt = q[b : b + 1].transpose(1, 2)
        out[b : b + 1] = torch.nn.functional.scaled_dot_product_attention(
            qt, kt, vt, is_causal=False, scale=scale).transpose(1, 2)
    return out


def prefill_literal(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """The reference's prefill, statement by statement (flex_backend.py:144-185)."""
    n_rep = q.shape[2] // k.shape[2]
    qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    if n_rep > 1:
        kt = kt.repeat_interleave(n_rep, dim=1)
        vt = vt.repeat_interleave(n_rep, dim=1)
    return torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, is_causal=True, scale=scale).transpose(1, 2)


# --------------------------------------------------------------------------- fp8 e4m3 pool


def quantize_kv_e4m3(pool: torch.Tensor, block_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-(block, kv head) absmax quantisation to OCP e4m3fn.

    pool ``[num_blocks*block_size, Hkv, D]`` (any float type) ->
    (``uint8`` bytes of the same shape, ``float32 [num_blocks, Hkv]`` scales)
    with scale = absmax/448 (1 for an all-zero tile) and byte = e4m3fn(x/scale),
    both divisions in fp32, conversion round-to-nearest-even (torch's).
    """
    slots, hkv, d = pool.shape
    nb = slots // block_size
    x = pool.to(torch.float32).reshape(nb, block_size, hkv, d)
    amax = x.abs().amax(dim=(1, 3))  # [nb, hkv]
    scale = torch.where(amax > 0, amax / torch.tensor(448.0, dtype=torch.float32), torch.ones_like(amax))
    y = (x / scale[:, None, :, None]).to(torch.float8_e4m3fn)
    return y.reshape(slots, hkv, d).view(torch.uint8), scale


def dequantize_kv_e4m3(bits: torch.Tensor, scale: torch.Tensor, block_size: int) -> torch.Tensor:
    """float32 pool from e4m3fn bytes and per-(block, head) scales."""
    slots, hkv, d = bits.shape
    nb = slots // block_size
    x = bits.view(torch.float8_e4m3fn).to(torch.float32).reshape(nb, block_size, hkv, d)
    return (x * scale[:, None, :, None]).reshape(slots, hkv, d)


def append_kv_e4m3(bits: torch.Tensor, scale: torch.Tensor, src: torch.Tensor, slots, block_size: int) -> None:
    """Append rows to an fp8 pool in place, "re-round on growth" (not a reference function: the reference has no
    fp8 pool; this states the policy the HIP entry point pa_kv_append_e4m3 documents, tile by tile in fp32).

    bits ``uint8 [total_slots, Hkv, D]``, scale ``float32 [num_blocks, Hkv]``, src ``[N, Hkv, D]``.  Per (block,
    kv head) tile: rows below the lowest offset written by this call are the content so far;
    a_old = scale*max|content|, a_new = max|new rows|; if a_new > a_old (or offset 0 is written) the scale becomes
    a_new/448 (1 for 0) and the content is re-rounded as e4m3(float(byte)*(scale/scale')); new rows are
    e4m3(x/scale').  Pinned by: appending a whole block at once equals quantize_kv_e4m3 of that block; appending
    rows of non-increasing magnitude never changes earlier bytes; the dequantised error bound in the tests.
    """
    f8 = torch.float8_e4m3fn
    slots = np.asarray(slots, dtype=np.int64)
    total_slots, hkv, d = bits.shape
    nb = total_slots // block_size
    x = src.to(torch.float32)
    c448 = torch.tensor(448.0, dtype=torch.float32)
    by_block = {}
    for t, s in enumerate(slots):
        if 0 <= s < nb * block_size:
            by_block.setdefault(int(s // block_size), {})[int(s % block_size)] = t  # later token wins
    for blk, offs in by_block.items():
        first = min(offs)
        rows = sorted(offs)
        toks = [offs[o] for o in rows]
        for h in range(hkv):
            s_old = scale[blk, h].clone()
            content = bits[blk * block_size : blk * block_size + first, h].view(f8).to(torch.float32)
            new = x[toks, h]
            a_new = new.abs().amax() if new.numel() else torch.tensor(0.0)
            a_old = s_old * content.abs().amax() if first > 0 else torch.tensor(0.0)
            s_new = s_old
            if first == 0 or a_new > a_old:
                s_new = a_new / c448 if a_new > 0 else torch.tensor(1.0, dtype=torch.float32)
            if first > 0 and s_new != s_old:
                ratio = s_old / s_new
                bits[blk * block_size : blk * block_size + first, h] = (content * ratio).to(f8).view(torch.uint8)
            enc = (new / s_new).to(f8).view(torch.uint8)
            for i, o in enumerate(rows):
                bits[blk * block_size + o, h] = enc[i]
            scale[blk, h] = s_new
