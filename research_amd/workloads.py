"""Seeded synthetic workloads for the paged-attention path.

Five named configurations, generated with ``numpy.random.default_rng(seed)``
(PCG64; the stream does not depend on the numpy version) so that the CPU
checker, the CPU baseline and the GPU kernels see identical inputs:

* ``c1`` fp32 decode, B=4, Hq=8, Hkv=2, D=64, lengths uniform in [1, 256],
  pool of 128 blocks                                             (seed 1001)
* ``c2`` bf16 decode, B=64, Hq=16, Hkv=8, D=128, lengths uniform in
  [512, 4096], pool sized to the blocks in use                   (seed 1002)
* ``c3`` bf16 chunked prefill + KV append, 32 sequences sharing a 2048-token
  prefix (same block ids) with a 256-token private chunk each,
  Hq=32, Hkv=8, D=128, pool of 640 blocks                        (seed 1003)
* ``c4`` bf16 decode, B=256, Hq=32, Hkv=8, D=128, lengths
  clip(rint(exp(N(ln 2048, 1))), 64, 32768)                      (seed 1004)
* ``c5`` fp8-e4m3 decode, B=8, Hq=32, Hkv=8, D=128, lengths uniform in
  [65536, 131072], per-(block, head) absmax scales                (seed 1005)

block_size is 16 everywhere.  Draw order is fixed: lengths, pool permutation,
q, k, v; values are N(0,1) in fp32, cast once to the target type.  Block
tables are consecutive slices of the permutation.  Every generator takes
overrides (``batch``, ``len_range`` ...) so that tests can run the same
construction at sizes a CPU checker finishes quickly.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import numpy as np
import torch

BLOCK_SIZE = 16
SEEDS = {"c1": 1001, "c2": 1002, "c3": 1003, "c4": 1004, "c5": 1005}


@dataclass
class DecodeWorkload:
    name: str
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    block_size: int
    num_blocks: int
    seq_lens: np.ndarray            # int64 [B]
    block_tables: List[np.ndarray]  # per sequence, int64 block ids
    q: torch.Tensor                 # [B, Hq, D] in `dtype`
    k_pool: torch.Tensor            # [num_blocks*block_size, Hkv, D] in `dtype` (full precision, also for fp8)
    v_pool: torch.Tensor
    dtype: torch.dtype
    kv_format: Optional[str] = None  # None or "fp8_e4m3"
    scale: float = 0.0
    tolerance: float = 0.0

    @property
    def batch(self) -> int:
        return len(self.seq_lens)

    @property
    def total_tokens(self) -> int:
        return int(self.seq_lens.sum())

    def padded_tables(self) -> np.ndarray:
        width = max((len(t) for t in self.block_tables), default=1)
        out = np.full((self.batch, max(width, 1)), -1, dtype=np.int32)
        for i, t in enumerate(self.block_tables):
            out[i, : len(t)] = t
        return out

    def algorithmic_bytes(self) -> int:
        """Bytes a decode step must move: every K/V byte once, q, out, tables, lengths (+ fp8 scales)."""
        kv_size = 1 if self.kv_format == "fp8_e4m3" else self.q.element_size()
        blocks = int(sum(len(t) for t in self.block_tables))
        n = self.total_tokens * self.num_kv_heads * self.head_dim * 2 * kv_size
        n += self.batch * self.num_q_heads * self.head_dim * 2 * self.q.element_size()
        n += blocks * 4 + self.batch * 4
        if self.kv_format == "fp8_e4m3":
            n += blocks * self.num_kv_heads * 2 * 4
        return n


@dataclass
class PrefillWorkload:
    name: str
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    block_size: int
    num_blocks: int
    prefix_len: int
    chunk_len: int
    block_tables: List[np.ndarray]  # per sequence: shared prefix blocks then private blocks
    q: torch.Tensor                 # [S, C, Hq, D]
    k_chunk: torch.Tensor           # [S, C, Hkv, D]
    v_chunk: torch.Tensor
    k_prefix: torch.Tensor          # [P, Hkv, D]
    v_prefix: torch.Tensor
    dtype: torch.dtype
    scale: float = 0.0
    tolerance: float = 0.0

    @property
    def num_seqs(self) -> int:
        return self.q.shape[0]

    def prefix_slots(self) -> np.ndarray:
        return _slots(self.block_tables[0], np.arange(self.prefix_len), self.block_size)

    def chunk_slots(self) -> np.ndarray:
        """slot_mapping of the append: positions P..P+C-1 of every sequence, sequence-major."""
        pos = np.arange(self.prefix_len, self.prefix_len + self.chunk_len)
        return np.concatenate([_slots(t, pos, self.block_size) for t in self.block_tables])

    def append_bytes(self) -> int:
        n = self.num_seqs * self.chunk_len
        return n * self.num_kv_heads * self.head_dim * 2 * 2 * self.q.element_size() + n * 8

    def attention_flops(self) -> int:
        """4*D*Hq*sum over chunk rows of the keys each row attends (causal-exact)."""
        keys = sum(self.prefix_len + i + 1 for i in range(self.chunk_len))
        return 4 * self.head_dim * self.num_q_heads * keys * self.num_seqs


def _slots(table: np.ndarray, pos: np.ndarray, block_size: int) -> np.ndarray:
    return np.asarray(table, dtype=np.int64)[pos // block_size] * block_size + pos % block_size


def _normal(rng: np.random.Generator, shape) -> np.ndarray:
    return rng.standard_normal(shape, dtype=np.float32)


def _cast(x: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    t = torch.from_numpy(x)
    return t if dtype == torch.float32 else t.to(dtype)


def _tables_from(perm: np.ndarray, seq_lens: np.ndarray, block_size: int) -> List[np.ndarray]:
    counts = -(-seq_lens // block_size)
    ends = np.cumsum(counts)
    return [perm[e - c : e].astype(np.int64) for c, e in zip(counts, ends)]


def _fill_pool(rng, tables, seq_lens, num_blocks, block_size, hkv, d, dtype) -> torch.Tensor:
    """Draw N(0,1) rows for every token in sequence order and place them in their slots."""
    pool = torch.zeros((num_blocks * block_size, hkv, d), dtype=dtype)
    for table, n in zip(tables, seq_lens):
        n = int(n)
        if n == 0:
            continue
        rows = _cast(_normal(rng, (n, hkv, d)), dtype)
        pool[torch.from_numpy(_slots(table, np.arange(n), block_size))] = rows
    return pool


def make_decode(
    name: str,
    batch: Optional[int] = None,
    len_range: Optional[Tuple[int, int]] = None,
    num_blocks: Optional[int] = None,
    seed: Optional[int] = None,
) -> DecodeWorkload:
    """Build decode configuration ``c1``, ``c2``, ``c4`` or ``c5`` (optionally scaled down)."""
    spec = {
        # name: (B, Hq, Hkv, D, dtype, kv_format, tolerance)
        "c1": (4, 8, 2, 64, torch.float32, None, 1e-5),
        "c2": (64, 16, 8, 128, torch.bfloat16, None, 2e-2),
        "c4": (256, 32, 8, 128, torch.bfloat16, None, 2e-2),
        "c5": (8, 32, 8, 128, torch.bfloat16, "fp8_e4m3", 6e-2),
    }[name]
    b, hq, hkv, d, dtype, kv_format, tol = spec
    b = batch if batch is not None else b
    rng = np.random.default_rng(SEEDS[name] if seed is None else seed)
    bs = BLOCK_SIZE
    if name == "c4":
        lo, hi = len_range or (64, 32768)
        lens = np.clip(np.rint(np.exp(rng.normal(np.log(2048.0), 1.0, b))), lo, hi).astype(np.int64)
    else:
        lo, hi = len_range or {"c1": (1, 256), "c2": (512, 4096), "c5": (65536, 131072)}[name]
        lens = rng.integers(lo, hi + 1, b).astype(np.int64)
    used = int((-(-lens // bs)).sum())
    if num_blocks is None:
        num_blocks = 128 if name == "c1" else used
    assert used <= num_blocks, "pool too small for the drawn lengths"
    perm = rng.permutation(num_blocks)
    tables = _tables_from(perm, lens, bs)
    q = _cast(_normal(rng, (b, hq, d)), dtype)
    k_pool = _fill_pool(rng, tables, lens, num_blocks, bs, hkv, d, dtype)
    v_pool = _fill_pool(rng, tables, lens, num_blocks, bs, hkv, d, dtype)
    return DecodeWorkload(
        name=name, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, block_size=bs, num_blocks=num_blocks,
        seq_lens=lens, block_tables=tables, q=q, k_pool=k_pool, v_pool=v_pool, dtype=dtype, kv_format=kv_format,
        scale=d**-0.5, tolerance=tol,
    )


def make_prefill_c3(
    num_seqs: int = 32,
    prefix_len: int = 2048,
    chunk_len: int = 256,
    num_q_heads: int = 32,
    num_kv_heads: int = 8,
    head_dim: int = 128,
    num_blocks: Optional[int] = None,
    dtype: torch.dtype = torch.bfloat16,
    seed: Optional[int] = None,
) -> PrefillWorkload:
    """Configuration ``c3``: shared-prefix chunked prefill (optionally scaled down)."""
    bs = BLOCK_SIZE
    assert prefix_len % bs == 0, "the shared prefix must end on a block boundary"
    shared = prefix_len // bs
    own = -(-chunk_len // bs)
    need = shared + num_seqs * own
    num_blocks = need if num_blocks is None else num_blocks
    assert need <= num_blocks
    rng = np.random.default_rng(SEEDS["c3"] if seed is None else seed)
    perm = rng.permutation(num_blocks).astype(np.int64)
    tables = [np.concatenate([perm[:shared], perm[shared + i * own : shared + (i + 1) * own]]) for i in range(num_seqs)]
    q = _cast(_normal(rng, (num_seqs, chunk_len, num_q_heads, head_dim)), dtype)
    k_prefix = _cast(_normal(rng, (prefix_len, num_kv_heads, head_dim)), dtype)
    k_chunk = _cast(_normal(rng, (num_seqs, chunk_len, num_kv_heads, head_dim)), dtype)
    v_prefix = _cast(_normal(rng, (prefix_len, num_kv_heads, head_dim)), dtype)
    v_chunk = _cast(_normal(rng, (num_seqs, chunk_len, num_kv_heads, head_dim)), dtype)
    return PrefillWorkload(
        name="c3", num_q_heads=num_q_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, block_size=bs,
        num_blocks=num_blocks, prefix_len=prefix_len, chunk_len=chunk_len, block_tables=tables, q=q,
        k_chunk=k_chunk, v_chunk=v_chunk, k_prefix=k_prefix, v_prefix=v_prefix, dtype=dtype,
        scale=head_dim**-0.5, tolerance=1e-5 if dtype == torch.float32 else 2e-2,
    )
