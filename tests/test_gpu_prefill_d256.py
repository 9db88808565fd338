"""Causal prefill with head_dim 256 on the GPU: the matrix-core kernel for that head size (one 32-row task per
wave, 32-key ring stages, table-driven loads) against the CPU checker and, for the zero-row rule of absent
blocks, against the vector kernel."""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import ops
from tests.gpu_helpers import DEV, announce, assert_close, tables_to_device

pytestmark = pytest.mark.gpu

D = 256


def _i32(x):
    return torch.tensor(list(x), dtype=torch.int32, device=DEV)


def _randn(rng, shape, dtype, scale=1.0):
    return (scale * torch.from_numpy(rng.standard_normal(shape).astype(np.float32))).to(dtype)


def _pool(rng, prefix, chunk, bs, hkv, dtype, spare=3):
    need = [-(-(p + c) // bs) for p, c in zip(prefix, chunk)]
    nb = sum(need) + spare
    perm = rng.permutation(nb)
    tables, at = [], 0
    for n in need:
        tables.append(perm[at : at + n].tolist())
        at += n
    kc = _randn(rng, (nb * bs, hkv, D), dtype)
    vc = _randn(rng, (nb * bs, hkv, D), dtype)
    return tables, kc, vc, nb


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv", [(4, 4), (6, 2), (8, 1)])
def test_shapes_and_block_sizes(dtype, hq, hkv):
    """Ragged chunks and prefixes (chunks of 1 row, of one and of several row blocks; prefixes that end inside a
    32-key stage) for block sizes the matrix-core kernel takes (16, 64, 96) and two it leaves to the vector
    kernel (8, 5), with group sizes 1, 3 and 8 (the four waves of a workgroup then hold different row blocks,
    one row block and three heads, or four heads of one row block)."""
    announce(f"prefill d256 shapes {dtype} hq={hq} hkv={hkv}")
    rng = np.random.default_rng(900 + hq)
    for bs in (16, 64, 96, 8, 5):
        prefix = [0, 130, 67, 300, 1]
        chunk = [70, 33, 129, 1, 64]
        cmax = max(chunk)
        tables, kc, vc, _ = _pool(rng, prefix, chunk, bs, hkv, dtype)
        q = _randn(rng, (len(chunk), cmax, hq, D), dtype)
        want = po.paged_prefill_chunk(q, kc, vc, tables, prefix, chunk, bs, D ** -0.5)
        out = torch.zeros(len(chunk) * cmax, hq, D, device=DEV, dtype=dtype)
        ops.prefill_paged(q.reshape(-1, hq, D).to(DEV), kc.to(DEV), vc.to(DEV), tables_to_device(tables),
                          _i32([p + c for p, c in zip(prefix, chunk)]), _i32(chunk), _i32(np.arange(len(chunk)) * cmax),
                          cmax, bs, D ** -0.5, out=out)
        assert_close(out.reshape(len(chunk), cmax, hq, D), want, 2e-2, f"block_size {bs}")


def test_dense_rows_documents_and_windows():
    """Dense rows handed over as one block per sequence whose length (700) is not a multiple of 16: the last
    16-key group of a sequence runs into the next sequence's rows, and the pool's last group past the end of the
    pool.  With per-row first keys (packed documents, attention/mask.py:141-191), a sliding window, both, and
    neither."""
    announce("prefill d256 dense, documents and windows")
    rng = np.random.default_rng(901)
    hq, hkv, b, t = 8, 2, 2, 700
    q, k, v = (_randn(rng, (b, t, h, D), torch.bfloat16) for h in (hq, hkv, hkv))
    ident = torch.arange(b, dtype=torch.int32, device=DEV).reshape(b, 1).contiguous()
    lens = _i32([t] * b)
    for doc_lens in (None, (1, 31, 32, 0, 64, 65, 300, 150), (333, 300)):
        first = None
        if doc_lens is not None:
            bounds = np.asarray(po.document_boundaries(doc_lens))
            first = bounds[np.searchsorted(bounds[1:], np.arange(t), side="right")].astype(np.int32)
            first = torch.from_numpy(np.tile(first, b)).to(DEV)
        for window in (0, 40):
            got = ops.prefill_paged(q.reshape(b * t, hq, D).to(DEV), k.reshape(b * t, hkv, D).to(DEV),
                                    v.reshape(b * t, hkv, D).to(DEV), ident, lens, lens, _i32(np.arange(b) * t), t, t,
                                    D ** -0.5, window=window, row_first_key=first)
            want = po.dense_prefill(q, k, v, D ** -0.5, window=window, doc_lens=doc_lens)
            assert_close(got.reshape(b, t, hq, D), want, 2e-2, f"documents {doc_lens} window {window}")


def test_sliding_window_over_a_long_prefix():
    """Windows much shorter than the prefix: workgroups start deep inside the context (the ring starts at an
    arbitrary stage), for 16-token blocks and for whole-sequence blocks."""
    announce("prefill d256 window, long prefix")
    rng = np.random.default_rng(902)
    hq, hkv = 8, 2
    for bs in (16, 2048):
        prefix, chunk = [1500, 1111, 0], [300, 77, 260]
        cmax = max(chunk)
        tables, kc, vc, _ = _pool(rng, prefix, chunk, bs, hkv, torch.bfloat16, spare=1)
        q = _randn(rng, (3, cmax, hq, D), torch.bfloat16)
        for window in (33, 64, 200, 1100):
            want = po.paged_prefill_chunk(q, kc, vc, tables, prefix, chunk, bs, D ** -0.5, window=window)
            out = torch.zeros(3 * cmax, hq, D, device=DEV, dtype=torch.bfloat16)
            ops.prefill_paged(q.reshape(-1, hq, D).to(DEV), kc.to(DEV), vc.to(DEV), tables_to_device(tables),
                              _i32([p + c for p, c in zip(prefix, chunk)]), _i32(chunk), _i32(np.arange(3) * cmax),
                              cmax, bs, D ** -0.5, out=out, window=window)
            assert_close(out.reshape(3, cmax, hq, D), want, 2e-2, f"block_size {bs} window {window}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_absent_blocks_and_short_tables(dtype):
    """Block ids of -1 or past the pool, and contexts longer than the table, stand for zero key / value rows
    there as in the vector kernel (which is the statement of that rule: flex_backend.py:272-277 leaves rows of
    absent blocks zero); the two kernels must agree on every row, for 16-token and 64-token blocks, with the bad
    entries in the first stage, in the middle and at the end."""
    announce(f"prefill d256 absent blocks {dtype}")
    rng = np.random.default_rng(903)
    hq, hkv = 8, 2
    for bs in (16, 64):
        prefix = [200, 0, 333, 64]
        chunk = [100, 190, 31, 64]
        cmax = max(chunk)
        tables, kc, vc, nb = _pool(rng, prefix, chunk, bs, hkv, dtype, spare=2)
        need = [len(t) for t in tables]
        tables[0][0] = -1                 # first stage
        tables[0][need[0] // 2] = nb + 5  # past the pool
        tables[1][-1] = -1                # last block
        tables[2] = tables[2][: need[2] - 2]  # table shorter than the context
        width = max(len(t) for t in tables)
        dev_tables = torch.tensor([t + [-1] * (width - len(t)) for t in tables], dtype=torch.int32, device=DEV)
        q = _randn(rng, (len(chunk) * cmax, hq, D), dtype).to(DEV)
        args = (q, kc.to(DEV), vc.to(DEV), dev_tables, _i32([p + c for p, c in zip(prefix, chunk)]), _i32(chunk),
                _i32(np.arange(len(chunk)) * cmax), cmax, bs, D ** -0.5)
        got = ops.prefill_paged(*args).float().cpu().reshape(len(chunk), cmax, hq, D)
        want = ops.prefill_paged(*args, rowwise=True).float().cpu().reshape(len(chunk), cmax, hq, D)
        for b, c in enumerate(chunk):
            assert_close(got[b, :c], want[b, :c], 2e-2, f"block_size {bs} sequence {b}")


def test_long_context_and_table_refills():
    """A 70 000-key context (4 375 slot-table entries) through the matrix-core kernel; contexts longer than what
    its LDS tables hold of them (the kernel fills the tables again every 3 064 tiles of 32 keys: one refill, and
    two refills with blocks missing on either side of the second); a table cut short of the context (the keys past
    it are absent); a window that starts the workgroup far into such a context; and a context that is one block of
    a length that is no multiple of 16, whose last group lies in the third fill.  All against the vector kernel
    on the chunk's rows."""
    announce("prefill d256 long context")
    rng = np.random.default_rng(904)
    hq, hkv, bs = 4, 1, 16
    seg = 3064 * 32  # keys per fill of the tables
    for ctx, table_len, window in ((70000, None, 0), (6144 * 16 + 40, None, 0), (6144 * 16 + 40, 6144, 0),
                                   (2 * seg + 5000, None, 0), (2 * seg + 5000, None, seg + 7000)):
        chunk = 48
        nblk = -(-ctx // bs)
        kc = _randn(rng, (nblk * bs, hkv, D), torch.bfloat16).to(DEV)
        vc = _randn(rng, (nblk * bs, hkv, D), torch.bfloat16).to(DEV)
        q = _randn(rng, (chunk, hq, D), torch.bfloat16, 0.3).to(DEV)
        blocks = rng.permutation(nblk).astype(np.int32)[:table_len]
        if ctx > 2 * seg:  # blocks missing around the second refill, and one block id past the pool
            blocks[2 * seg // bs - 3 : 2 * seg // bs + 2] = -1
            blocks[seg // bs + 1] = nblk + 5
        table = torch.from_numpy(blocks).reshape(1, -1).contiguous().to(DEV)
        args = (q, kc, vc, table, _i32([ctx]), _i32([chunk]), _i32([0]), chunk, bs, D ** -0.5)
        got = ops.prefill_paged(*args, window=window).float().cpu()
        want = ops.prefill_paged(*args, window=window, rowwise=True).float().cpu()
        assert_close(got, want, 2e-2, f"context of {ctx} keys, table of {table.shape[1]} entries, window {window}")
    # per-row first keys over the last of these contexts: a document that starts at key 1000, then one that starts
    # with row 20
    first = torch.tensor([1000] * 20 + [ctx - chunk + 20] * (chunk - 20), dtype=torch.int32, device=DEV)
    got = ops.prefill_paged(*args, row_first_key=first).float().cpu()
    want = ops.prefill_paged(*args, row_first_key=first, rowwise=True).float().cpu()
    assert_close(got, want, 2e-2, f"context of {ctx} keys, per-row first keys")
    ctx, chunk = 2 * seg + 1111, 48
    kc = _randn(rng, (ctx, hkv, D), torch.bfloat16).to(DEV)
    vc = _randn(rng, (ctx, hkv, D), torch.bfloat16).to(DEV)
    q = _randn(rng, (chunk, hq, D), torch.bfloat16, 0.3).to(DEV)
    args = (q, kc, vc, torch.zeros(1, 1, dtype=torch.int32, device=DEV), _i32([ctx]), _i32([chunk]), _i32([0]), chunk, ctx, D ** -0.5)
    got = ops.prefill_paged(*args).float().cpu()
    want = ops.prefill_paged(*args, rowwise=True).float().cpu()
    assert_close(got, want, 2e-2, f"one block of {ctx} keys")


def test_c3_shape_at_head_dim_256_full_size():
    """The chunked-prefill workload's shape (32 x (2048 shared + 256 own) tokens, 16-token blocks) with 16 query /
    8 kv heads of 256: every output element against the vector kernel, and all 32 sequences against the
    checker."""
    from research_amd.workloads import make_prefill_c3

    announce("prefill d256, c3 shape, full size")
    w = make_prefill_c3(num_q_heads=16, num_kv_heads=8, head_dim=D, seed=905)
    S, C, P = w.num_seqs, w.chunk_len, w.prefix_len
    shape = (w.num_blocks * w.block_size, w.num_kv_heads, D)
    kc = torch.zeros(shape, dtype=w.dtype, device=DEV)
    vc = torch.zeros_like(kc)
    ops.kv_scatter(kc, vc, w.k_prefix.to(DEV), w.v_prefix.to(DEV), torch.from_numpy(w.prefix_slots()).to(DEV))
    ops.kv_scatter(kc, vc, w.k_chunk.reshape(S * C, *shape[1:]).to(DEV), w.v_chunk.reshape(S * C, *shape[1:]).to(DEV),
                   torch.from_numpy(w.chunk_slots()).to(DEV))
    q = w.q.reshape(S * C, w.num_q_heads, D).to(DEV)
    args = (q, kc, vc, tables_to_device(w.block_tables), _i32([P + C] * S), _i32([C] * S), _i32(np.arange(S) * C), C,
            w.block_size, w.scale)
    mfma = ops.prefill_paged(*args).float().cpu()
    rowwise = ops.prefill_paged(*args, rowwise=True).float().cpu()
    assert_close(mfma, rowwise, 2e-2, "matrix-core kernel against the vector kernel, all rows")
    seqs = list(range(S))
    want = po.paged_prefill_chunk(w.q[seqs], kc.cpu(), vc.cpu(), [w.block_tables[s] for s in seqs], [P] * S, [C] * S,
                                  w.block_size, w.scale)
    assert_close(mfma.reshape(S, C, w.num_q_heads, D), want, 2e-2, "against the checker, all sequences")
