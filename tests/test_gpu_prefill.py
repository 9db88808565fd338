"""Causal prefill on the GPU against the CPU checker: the dense case the
reference has (its own recipe and tolerance) and chunked prefill over shared
prefix blocks."""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import ops
from research_amd.workloads import make_prefill_c3
from tests.gpu_helpers import DEV, announce, assert_close, tables_to_device

pytestmark = pytest.mark.gpu


def _i32(x):
    return torch.tensor(list(x), dtype=torch.int32, device=DEV)


def _run_chunked(w, q=None):
    """Append prefix and chunks, then prefill every chunk over its prefix, all on the device."""
    shape = (w.num_blocks * w.block_size, w.num_kv_heads, w.head_dim)
    kc = torch.zeros(shape, dtype=w.dtype, device=DEV)
    vc = torch.zeros_like(kc)
    ops.kv_scatter(kc, vc, w.k_prefix.to(DEV), w.v_prefix.to(DEV), torch.from_numpy(w.prefix_slots()).to(DEV))
    ops.kv_scatter(kc, vc, w.k_chunk.reshape(-1, *shape[1:]).to(DEV), w.v_chunk.reshape(-1, *shape[1:]).to(DEV),
                   torch.from_numpy(w.chunk_slots()).to(DEV))
    S, C = w.num_seqs, w.chunk_len
    q = w.q if q is None else q
    out = ops.prefill_paged(q.reshape(S * C, w.num_q_heads, w.head_dim).to(DEV), kc, vc,
                            tables_to_device(w.block_tables), _i32([w.prefix_len + C] * S), _i32([C] * S),
                            _i32(np.arange(S) * C), C, w.block_size, w.scale)
    return out.reshape(S, C, w.num_q_heads, w.head_dim), kc, vc


def test_dense_prefill_reference_recipe():
    """B=2,T=8,Hq=4,Hkv=2,D=32 bf16, seed 42; bars max<0.01, mean<0.001 (test_kv_cache.py:276-345)."""
    announce("prefill reference recipe")
    torch.manual_seed(42)
    q = torch.randn(2, 8, 4, 32).to(torch.bfloat16)
    k = torch.randn(2, 8, 2, 32).to(torch.bfloat16)
    v = torch.randn(2, 8, 2, 32).to(torch.bfloat16)
    out = ops.prefill_paged(q.reshape(16, 4, 32).to(DEV), k.reshape(16, 2, 32).to(DEV), v.reshape(16, 2, 32).to(DEV),
                            _i32([0, 1]).reshape(2, 1), _i32([8, 8]), _i32([8, 8]), _i32([0, 8]), 8, 8, 32**-0.5)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2).repeat_interleave(2, 1), v.transpose(1, 2).repeat_interleave(2, 1),
        is_causal=True).transpose(1, 2)
    diff = (out.reshape(2, 8, 4, 32).cpu().float() - ref.float()).abs()
    assert diff.max() < 0.01 and diff.mean() < 0.001
    assert_close(out.reshape(2, 8, 4, 32), po.dense_prefill(q, k, v, 32**-0.5), 2e-2, "dense prefill")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2), (torch.float16, 2e-2)])
def test_chunked_prefill_small(dtype, tol):
    announce(f"chunked prefill small {dtype}")
    w = make_prefill_c3(num_seqs=3, prefix_len=48, chunk_len=21, num_q_heads=8, num_kv_heads=2, head_dim=64,
                        dtype=dtype)
    got, kc, vc = _run_chunked(w)
    want = po.paged_prefill_chunk(w.q, kc.cpu(), vc.cpu(), w.block_tables, [48] * 3, [21] * 3, w.block_size, w.scale)
    assert_close(got, want, tol, "chunked small")


def test_chunked_prefill_ragged_chunks_and_prefixes():
    announce("chunked prefill ragged")
    rng = np.random.default_rng(31)
    bs, nb, hq, hkv, d = 16, 40, 4, 2, 64
    prefix, chunk = [0, 32, 19], [17, 5, 30]
    cmax = 30
    perm = rng.permutation(nb)
    tables, at = [], 0
    for p, c in zip(prefix, chunk):
        n = -(-(p + c) // bs)
        tables.append(perm[at : at + n].tolist())
        at += n
    kc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32))
    vc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32))
    q = torch.from_numpy(rng.standard_normal((3, cmax, hq, d)).astype(np.float32))
    want = po.paged_prefill_chunk(q, kc, vc, tables, prefix, chunk, bs, 0.125)
    out = torch.zeros(3 * cmax, hq, d, device=DEV)
    ops.prefill_paged(q.reshape(3 * cmax, hq, d).to(DEV), kc.to(DEV), vc.to(DEV), tables_to_device(tables),
                      _i32([p + c for p, c in zip(prefix, chunk)]), _i32(chunk), _i32(np.arange(3) * cmax), cmax, bs,
                      0.125, out=out)
    assert_close(out.reshape(3, cmax, hq, d), want, 1e-5, "ragged chunks")


def test_c3_reduced_shared_prefix():
    """workload c3's head shape with 4 sequences sharing a 512-token prefix, 64-token chunks."""
    announce("chunked prefill c3 reduced")
    w = make_prefill_c3(num_seqs=4, prefix_len=512, chunk_len=64)
    got, kc, vc = _run_chunked(w)
    want = po.paged_prefill_chunk(w.q, kc.cpu(), vc.cpu(), w.block_tables, [512] * 4, [64] * 4, w.block_size, w.scale)
    assert_close(got, want, 2e-2, "c3 reduced")
    # equals rows [P:P+C] of full causal attention over prefix+chunk for one sequence
    s = 2
    full = po.dense_prefill(torch.cat([torch.zeros(512, 32, 128, dtype=w.dtype), w.q[s]])[None],
                            torch.cat([w.k_prefix, w.k_chunk[s]])[None], torch.cat([w.v_prefix, w.v_chunk[s]])[None],
                            w.scale)
    assert_close(got[s], full[0, 512:], 2e-2, "rows of the full-sequence prefill")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_sliding_window_prefill(dtype, tol):
    """Chunked and dense prefill under a sliding window (the vector kernel runs windowed calls)."""
    announce(f"prefill window {dtype}")
    w = make_prefill_c3(num_seqs=3, prefix_len=96, chunk_len=40, num_q_heads=8, num_kv_heads=2, head_dim=64,
                        dtype=dtype)
    shape = (w.num_blocks * w.block_size, w.num_kv_heads, w.head_dim)
    kc = torch.zeros(shape, dtype=dtype, device=DEV)
    vc = torch.zeros_like(kc)
    ops.kv_scatter(kc, vc, w.k_prefix.to(DEV), w.v_prefix.to(DEV), torch.from_numpy(w.prefix_slots()).to(DEV))
    ops.kv_scatter(kc, vc, w.k_chunk.reshape(-1, *shape[1:]).to(DEV), w.v_chunk.reshape(-1, *shape[1:]).to(DEV),
                   torch.from_numpy(w.chunk_slots()).to(DEV))
    S, C, P = w.num_seqs, w.chunk_len, w.prefix_len
    q = w.q.reshape(S * C, w.num_q_heads, w.head_dim).to(DEV)
    tables = tables_to_device(w.block_tables)
    for window in (1, 7, 40, 41, 130, 1000):
        got = ops.prefill_paged(q, kc, vc, tables, _i32([P + C] * S), _i32([C] * S), _i32(np.arange(S) * C), C,
                                w.block_size, w.scale, window=window).reshape(S, C, w.num_q_heads, w.head_dim)
        want = po.paged_prefill_chunk(w.q, kc.cpu(), vc.cpu(), w.block_tables, [P] * S, [C] * S, w.block_size,
                                      w.scale, window=window)
        assert_close(got, want, tol, f"chunked window {window}")
    # dense: the step's own K/V as a pool of S blocks of C tokens
    k = w.k_chunk.reshape(S * C, *shape[1:]).to(DEV)
    v = w.v_chunk.reshape(S * C, *shape[1:]).to(DEV)
    ident = torch.arange(S, dtype=torch.int32, device=DEV).reshape(S, 1).contiguous()
    got = ops.prefill_paged(q, k, v, ident, _i32([C] * S), _i32([C] * S), _i32(np.arange(S) * C), C, C, w.scale,
                            window=9).reshape(S, C, w.num_q_heads, w.head_dim)
    assert_close(got, po.dense_prefill(w.q, w.k_chunk, w.v_chunk, w.scale, window=9), tol, "dense window 9")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("hq,hkv", [(4, 4), (6, 2), (8, 1)])
def test_matrix_core_kernel_shapes_and_block_sizes(dtype, d, hq, hkv):
    """The matrix-core kernel over ragged chunks and prefixes for block sizes that take the scalar-base loads
    (16; 8, 64, 96 via the incremental walk) and one that makes loads straddle blocks (5), with group sizes
    1, 3 (odd: a wave's two column tiles are different row blocks) and 8."""
    announce(f"prefill mfma shapes {dtype} d={d} hq={hq} hkv={hkv}")
    rng = np.random.default_rng(100 + d + hq)
    for bs in (16, 8, 5, 64, 96):
        prefix = [0, 130, 67, 300, 1]
        chunk = [70, 33, 129, 1, 64]
        cmax = max(chunk)
        need = [-(-(p + c) // bs) for p, c in zip(prefix, chunk)]
        nb = sum(need) + 3
        perm = rng.permutation(nb)
        tables, at = [], 0
        for n in need:
            tables.append(perm[at : at + n].tolist())
            at += n
        kc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
        vc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
        q = torch.from_numpy(rng.standard_normal((len(chunk), cmax, hq, d)).astype(np.float32)).to(dtype)
        want = po.paged_prefill_chunk(q, kc, vc, tables, prefix, chunk, bs, d ** -0.5)
        out = torch.zeros(len(chunk) * cmax, hq, d, device=DEV, dtype=dtype)
        ops.prefill_paged(q.reshape(-1, hq, d).to(DEV), kc.to(DEV), vc.to(DEV), tables_to_device(tables),
                          _i32([p + c for p, c in zip(prefix, chunk)]), _i32(chunk), _i32(np.arange(len(chunk)) * cmax),
                          cmax, bs, d ** -0.5, out=out)
        assert_close(out.reshape(len(chunk), cmax, hq, d), want, 2e-2, f"block_size {bs}")


def test_sliding_window_prefill_long_prefix_on_the_matrix_core_kernel():
    """Windows much shorter than the prefix: workgroups start deep inside the context (ring and block-id window
    start at an arbitrary tile), for 16-token blocks and for whole-sequence blocks."""
    announce("prefill window, long prefix")
    rng = np.random.default_rng(77)
    hq, hkv, d = 8, 2, 128
    for bs in (16, 2048):
        prefix, chunk = [1500, 1111, 0], [300, 77, 260]
        cmax = max(chunk)
        need = [-(-(p + c) // bs) for p, c in zip(prefix, chunk)]
        nb = sum(need) + 1
        perm = rng.permutation(nb)
        tables, at = [], 0
        for n in need:
            tables.append(perm[at : at + n].tolist())
            at += n
        kc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16)
        vc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16)
        q = torch.from_numpy(rng.standard_normal((3, cmax, hq, d)).astype(np.float32)).to(torch.bfloat16)
        for window in (64, 65, 200, 513, 1100):
            want = po.paged_prefill_chunk(q, kc, vc, tables, prefix, chunk, bs, d ** -0.5, window=window)
            out = torch.zeros(3 * cmax, hq, d, device=DEV, dtype=torch.bfloat16)
            ops.prefill_paged(q.reshape(-1, hq, d).to(DEV), kc.to(DEV), vc.to(DEV), tables_to_device(tables),
                              _i32([p + c for p, c in zip(prefix, chunk)]), _i32(chunk), _i32(np.arange(3) * cmax),
                              cmax, bs, d ** -0.5, out=out, window=window)
            assert_close(out.reshape(3, cmax, hq, d), want, 2e-2, f"block_size {bs} window {window}")


@pytest.mark.parametrize("dtype,tol,d", [(torch.bfloat16, 2e-2, 128), (torch.float16, 2e-2, 64),
                                         (torch.float32, 1e-5, 64)])
def test_packed_documents_prefill(dtype, tol, d):
    """Per-row first keys: packed documents (attention/mask.py:141-191) in dense rows, with boundaries inside
    32-row blocks and 64-key tiles, an empty document, positions past the last document, alone and under a
    sliding window; bf16 / fp16 run on the matrix cores, fp32 on the vector kernel."""
    announce(f"prefill documents {dtype}")
    rng = np.random.default_rng(300 + d)
    hq, hkv, b, t = 8, 2, 2, 700
    q, k, v = (torch.from_numpy(rng.standard_normal((b, t, h, d)).astype(np.float32)).to(dtype)
               for h in (hq, hkv, hkv))
    ident = torch.arange(b, dtype=torch.int32, device=DEV).reshape(b, 1).contiguous()
    lens = _i32([t] * b)
    for doc_lens in ((700,), (1, 31, 32, 0, 64, 65, 300, 150), (333, 300), (5,) * 100):
        bounds = np.asarray(po.document_boundaries(doc_lens))
        first = bounds[np.searchsorted(bounds[1:], np.arange(t), side="right")].astype(np.int32)
        first = torch.from_numpy(np.tile(first, b)).to(DEV)
        for window in (0, 40):
            got = ops.prefill_paged(q.reshape(b * t, hq, d).to(DEV), k.reshape(b * t, hkv, d).to(DEV),
                                    v.reshape(b * t, hkv, d).to(DEV), ident, lens, lens, _i32(np.arange(b) * t), t, t,
                                    d ** -0.5, window=window, row_first_key=first)
            want = po.dense_prefill(q, k, v, d ** -0.5, window=window, doc_lens=doc_lens)
            assert_close(got.reshape(b, t, hq, d), want, tol, f"documents {doc_lens[:4]}.. window {window}")


def test_packed_documents_chunked_prefill_over_a_prefix():
    """Documents by absolute position in chunked prefill: the chunk's rows start inside a document that began
    in the cached prefix, 16-token blocks."""
    announce("prefill documents, chunked")
    rng = np.random.default_rng(311)
    hq, hkv, d, bs = 8, 2, 128, 16
    prefix, chunk = [500, 129], [200, 260]
    cmax = max(chunk)
    need = [-(-(p + c) // bs) for p, c in zip(prefix, chunk)]
    nb = sum(need) + 2
    perm = rng.permutation(nb)
    tables = [perm[: need[0]].tolist(), perm[need[0] : need[0] + need[1]].tolist()]
    kc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16)
    vc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16)
    q = torch.from_numpy(rng.standard_normal((2, cmax, hq, d)).astype(np.float32)).to(torch.bfloat16)
    doc_lens = (90, 350, 130, 47, 33, 200)
    bounds = np.asarray(po.document_boundaries(doc_lens))
    pos = np.asarray(prefix)[:, None] + np.arange(cmax)[None, :]
    first = bounds[np.searchsorted(bounds[1:], pos, side="right")].astype(np.int32)
    want = po.paged_prefill_chunk(q, kc, vc, tables, prefix, chunk, bs, d ** -0.5, doc_lens=doc_lens)
    out = torch.zeros(2 * cmax, hq, d, device=DEV, dtype=torch.bfloat16)
    ops.prefill_paged(q.reshape(-1, hq, d).to(DEV), kc.to(DEV), vc.to(DEV), tables_to_device(tables),
                      _i32([p + c for p, c in zip(prefix, chunk)]), _i32(chunk), _i32(np.arange(2) * cmax), cmax, bs,
                      d ** -0.5, out=out, row_first_key=torch.from_numpy(first.reshape(-1)).to(DEV))
    assert_close(out.reshape(2, cmax, hq, d), want, 2e-2, "chunked documents")


@pytest.mark.parametrize("d", [128, 64, 32])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_assembly_loop_kernel_absent_blocks_and_short_tables(dtype, d):
    """head_dim 128, 64 and 32 take the kernel whose tile loop is scheduled assembly.  Block ids of -1 or past the pool, and
    contexts longer than the table, stand for zero key / value rows there as in the vector kernel (which is the
    statement of that rule: flex_backend.py:272-277 leaves rows of absent blocks zero); the two kernels must
    agree on every row, for 16-token and 64-token blocks, with the bad entries in the first tile, in the middle
    and at the end."""
    announce(f"prefill assembly loop, absent blocks {dtype} d={d}")
    rng = np.random.default_rng(77)
    hq, hkv = 8, 2
    for bs in (16, 64):
        prefix = [200, 0, 333, 64]
        chunk = [100, 190, 31, 64]
        cmax = max(chunk)
        need = [-(-(p + c) // bs) for p, c in zip(prefix, chunk)]
        nb = sum(need) + 2
        perm = rng.permutation(nb)
        tables, at = [], 0
        for n in need:
            tables.append(perm[at : at + n].tolist())
            at += n
        tables[0][0] = -1               # first tile
        tables[0][need[0] // 2] = nb + 5  # past the pool
        tables[1][-1] = -1              # last block
        tables[2] = tables[2][: need[2] - 2]  # table shorter than the context
        width = max(len(t) for t in tables)
        dev_tables = torch.tensor([t + [-1] * (width - len(t)) for t in tables], dtype=torch.int32, device=DEV)
        kc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype).to(DEV)
        vc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype).to(DEV)
        q = torch.from_numpy(rng.standard_normal((len(chunk) * cmax, hq, d)).astype(np.float32)).to(dtype).to(DEV)
        args = (q, kc, vc, dev_tables, _i32([p + c for p, c in zip(prefix, chunk)]), _i32(chunk),
                _i32(np.arange(len(chunk)) * cmax), cmax, bs, d ** -0.5)
        for window in (0, 70):  # (with a window: the instance of the kernel that applies lower bounds)
            got = ops.prefill_paged(*args, window=window).float().cpu().reshape(len(chunk), cmax, hq, d)
            want = ops.prefill_paged(*args, window=window, rowwise=True).float().cpu().reshape(len(chunk), cmax, hq, d)
            for b, c in enumerate(chunk):
                assert_close(got[b, :c], want[b, :c], 2e-2, f"block_size {bs} sequence {b} window {window}")


@pytest.mark.parametrize("d", [128, 64, 32])
def test_assembly_loop_kernel_long_context_and_table_limit(d):
    """A 70 000-key context (more than a thousand tiles of slot-table entries) through the assembly-loop kernel,
    and a table just past what that kernel's LDS tables hold (the instance that fills its tables again runs;
    under a sliding window the other instance, its tables starting at the workgroup's first tile): both against
    the vector kernel on the chunk's rows."""
    announce(f"prefill assembly loop, long context d={d}")
    rng = np.random.default_rng(78)
    hq, hkv, bs = 4, 1, 16
    cap_tiles = 1600 if d == 128 else 4096  # tiles of 64 keys the kernel's slot tables hold at this head size
    for ctx in (70000, cap_tiles * 64 + 40):
        chunk = 48
        nblk = -(-ctx // bs)
        kc = torch.from_numpy(rng.standard_normal((nblk * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16).to(DEV)
        vc = torch.from_numpy(rng.standard_normal((nblk * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16).to(DEV)
        q = (0.3 * torch.from_numpy(rng.standard_normal((chunk, hq, d)).astype(np.float32))).to(torch.bfloat16).to(DEV)
        table = torch.from_numpy(rng.permutation(nblk).astype(np.int32)).reshape(1, -1).to(DEV)
        args = (q, kc, vc, table, _i32([ctx]), _i32([chunk]), _i32([0]), chunk, bs, d ** -0.5)
        for window in (0, 3000):  # (with a window the workgroup starts more than a thousand tiles into the tables)
            got = ops.prefill_paged(*args, window=window).float().cpu()
            want = ops.prefill_paged(*args, window=window, rowwise=True).float().cpu()
            assert_close(got, want, 2e-2, f"context of {ctx} keys, window {window}")


@pytest.mark.parametrize("d", [128, 64, 32])
def test_assembly_loop_kernel_table_refills(d):
    """Contexts longer than what the kernel's LDS tables hold of them (it fills them again every 1 596 tiles of 64
    keys at head_dim 128, every 4 092 below): two refills with blocks missing on either side of the second and one block id past the pool;
    a window that starts the workgroup far into such a context; and a context that is one block of a length that
    is no multiple of 16, whose last group lies in the third fill.  Against the vector kernel on the chunk's rows."""
    announce(f"prefill assembly loop, table refills d={d}")
    rng = np.random.default_rng(81)
    hq, hkv, bs, chunk = 4, 1, 16, 80
    seg = (1596 if d == 128 else 4092) * 64  # keys per fill of the tables
    mk = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(torch.bfloat16).to(DEV)
    ctx = 2 * seg + 5000
    nblk = -(-ctx // bs)
    blocks = rng.permutation(nblk).astype(np.int32)
    blocks[2 * seg // bs - 3 : 2 * seg // bs + 2] = -1
    blocks[seg // bs + 1] = nblk + 5
    table = torch.from_numpy(blocks).reshape(1, -1).contiguous().to(DEV)
    args = (0.3 * mk(chunk, hq, d), mk(nblk * bs, hkv, d), mk(nblk * bs, hkv, d), table, _i32([ctx]), _i32([chunk]), _i32([0]),
            chunk, bs, d ** -0.5)
    for window in (0, seg + 7000):
        got = ops.prefill_paged(*args, window=window).float().cpu()
        want = ops.prefill_paged(*args, window=window, rowwise=True).float().cpu()
        assert_close(got, want, 2e-2, f"context of {ctx} keys, window {window}")
    # per-row first keys: the chunk's first half belongs to a document that starts at key 1000, the rest to one that
    # starts with row 40
    first = torch.tensor([1000] * 40 + [ctx - chunk + 40] * (chunk - 40), dtype=torch.int32, device=DEV)
    got = ops.prefill_paged(*args, row_first_key=first).float().cpu()
    want = ops.prefill_paged(*args, row_first_key=first, rowwise=True).float().cpu()
    assert_close(got, want, 2e-2, f"context of {ctx} keys, per-row first keys")
    ctx = 2 * seg + 1111
    args = (0.3 * mk(chunk, hq, d), mk(ctx, hkv, d), mk(ctx, hkv, d), torch.zeros(1, 1, dtype=torch.int32, device=DEV), _i32([ctx]),
            _i32([chunk]), _i32([0]), chunk, ctx, d ** -0.5)
    got = ops.prefill_paged(*args).float().cpu()
    want = ops.prefill_paged(*args, rowwise=True).float().cpu()
    assert_close(got, want, 2e-2, f"one block of {ctx} keys")


@pytest.mark.parametrize("d", [256, 128, 64])
def test_assembly_loop_kernel_window_over_a_table_longer_than_its_tables(d):
    """Sliding window over contexts whose block table is longer than the kernel's slot tables: a chunk of 600 rows
    with one query head per kv head (a workgroup then spans the most rows it can), and the last 300 rows of a
    sequence whose context is one block of a length that is no multiple of 16; against the vector kernel."""
    announce(f"prefill assembly loop, window over a long table d={d}")
    rng = np.random.default_rng(80)
    cap_keys = {256: 6144 * 16, 128: 1600 * 64, 64: 4096 * 64}[d]  # keys the kernel's slot tables hold at this head size
    hq = hkv = 1
    mk = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(torch.bfloat16).to(DEV)
    ctx, chunk, bs = cap_keys + 5000, 600, 16
    nblk = -(-ctx // bs)
    table = torch.from_numpy(rng.permutation(nblk).astype(np.int32)).reshape(1, -1).to(DEV)
    args = (0.3 * mk(chunk, hq, d), mk(nblk * bs, hkv, d), mk(nblk * bs, hkv, d), table, _i32([ctx]), _i32([chunk]), _i32([0]),
            chunk, bs, d ** -0.5)
    for window in (1000, 1):
        got = ops.prefill_paged(*args, window=window).float().cpu()
        want = ops.prefill_paged(*args, window=window, rowwise=True).float().cpu()
        assert_close(got, want, 2e-2, f"paged, window {window}")
    t = cap_keys + 1111
    args = (0.3 * mk(300, hq, d), mk(t, hkv, d), mk(t, hkv, d), torch.zeros(1, 1, dtype=torch.int32, device=DEV), _i32([t]), _i32([300]),
            _i32([0]), 300, t, d ** -0.5)
    got = ops.prefill_paged(*args, window=500).float().cpu()
    want = ops.prefill_paged(*args, window=500, rowwise=True).float().cpu()
    assert_close(got, want, 2e-2, "one block of the whole context, window 500")


@pytest.mark.parametrize("d", [128, 64, 32])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_assembly_loop_kernel_dense_rows_of_any_length(dtype, d):
    """Dense rows handed over as one block per sequence whose length is not a multiple of 16 (what
    `_prefill_attention`, flex_backend.py:144-185, gets for an ordinary prompt): a sequence's last 16-key group
    runs into the next sequence's rows, and the last groups of the last sequences would run past the end of the
    pool (with 6-token sequences, two of the three sequences' only group).  With per-row first keys (packed
    documents, attention/mask.py:141-191), a sliding window, both, and neither; against the checker."""
    announce(f"prefill assembly loop, dense rows {dtype} d={d}")
    rng = np.random.default_rng(79)
    hq, hkv = 8, 2
    for b, t, doc_lens in ((2, 700, (1, 31, 32, 0, 64, 65, 300, 207)), (3, 6, (2, 4)), (1, 33, (33,)), (4, 129, (100, 29))):
        q, k, v = (torch.from_numpy(rng.standard_normal((b, t, h, d)).astype(np.float32)).to(dtype) for h in (hq, hkv, hkv))
        ident = torch.arange(b, dtype=torch.int32, device=DEV).reshape(b, 1).contiguous()
        lens = _i32([t] * b)
        bounds = np.asarray(po.document_boundaries(doc_lens))
        first = bounds[np.searchsorted(bounds[1:], np.arange(t), side="right")].astype(np.int32)
        first = torch.from_numpy(np.tile(first, b)).to(DEV)
        for docs in (None, doc_lens):
            for window in (0, 40):
                got = ops.prefill_paged(q.reshape(b * t, hq, d).to(DEV), k.reshape(b * t, hkv, d).to(DEV),
                                        v.reshape(b * t, hkv, d).to(DEV), ident, lens, lens, _i32(np.arange(b) * t), t, t,
                                        d ** -0.5, window=window, row_first_key=first if docs else None)
                want = po.dense_prefill(q, k, v, d ** -0.5, window=window, doc_lens=docs)
                assert_close(got.reshape(b, t, hq, d), want, 2e-2, f"{b} x {t}, documents {docs}, window {window}")


@pytest.mark.parametrize("d", [32, 64, 128, 256])
def test_one_short_block_per_sequence_and_a_longer_context(d):
    """One block per sequence that is not a multiple of 16 keys long, with contexts that run past it (the keys
    behind the block are absent: zero rows, as in the vector kernel, which states that rule) and chunks that do
    not start at key 0; the last sequence's block ends the pool.  Matrix-core kernels against the vector kernel."""
    announce(f"prefill, one short block per sequence d={d}")
    rng = np.random.default_rng(81 + d)
    hq, hkv = 4, 2
    for bs, ctx, chunk in ((33, [40, 33, 20], [40, 10, 20]), (100, [130, 100, 7], [60, 100, 7]), (17, [17, 30], [17, 30])):
        b = len(ctx)
        cmax = max(chunk)
        kc = torch.from_numpy(rng.standard_normal((b * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16).to(DEV)
        vc = torch.from_numpy(rng.standard_normal((b * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16).to(DEV)
        q = torch.from_numpy(rng.standard_normal((b * cmax, hq, d)).astype(np.float32)).to(torch.bfloat16).to(DEV)
        ident = torch.from_numpy(rng.permutation(b).astype(np.int32)).reshape(b, 1).contiguous().to(DEV)
        args = (q, kc, vc, ident, _i32(ctx), _i32(chunk), _i32(np.arange(b) * cmax), cmax, bs, d ** -0.5)
        for window in (0, 12):
            got = ops.prefill_paged(*args, window=window).float().cpu().reshape(b, cmax, hq, d)
            want = ops.prefill_paged(*args, window=window, rowwise=True).float().cpu().reshape(b, cmax, hq, d)
            for i, c in enumerate(chunk):
                assert_close(got[i, :c], want[i, :c], 2e-2, f"block_size {bs} sequence {i} window {window}")


@pytest.mark.parametrize("d", [32, 64, 128, 256])
def test_logits_that_grow_along_the_context(d):
    """Keys whose logits rise steeply with the key index (about 9 in base-2 units per 32 keys, from far below
    zero to far above), so that every row's reference maximum is outgrown by more than the lazy-rescale slack
    again and again, by some rows of a wave earlier than by others; then the same keys in falling order (the
    first subtile holds the maximum, nothing is ever rescaled).  The assembly loops of head_dim 32, 64, 128 and 256
    (and, with a window, their instances with lower bounds), chunked over a prefix, against the checker."""
    announce(f"prefill rescale paths d={d}")
    rng = np.random.default_rng(500 + d)
    hq, hkv, bs = 4, 2, 16
    prefix, chunk = [700, 0, 333], [200, 130, 64]
    cmax = max(chunk)
    need = [-(-(p + c) // bs) for p, c in zip(prefix, chunk)]
    nb = sum(need) + 1
    perm = rng.permutation(nb)
    tables, at = [], 0
    for n in need:
        tables.append(perm[at : at + n].tolist())
        at += n
    q = torch.from_numpy((rng.standard_normal((len(chunk), cmax, hq, d)) + 2.0).astype(np.float32)).to(torch.bfloat16)
    vc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16)
    for direction in (1, -1):
        kc = torch.zeros(nb * bs, hkv, d)
        for b, (p, c) in enumerate(zip(prefix, chunk)):
            n = p + c
            # natural-unit logit of key j for a row with sum(q) = 2d: about ramp[j]
            ramp = np.linspace(-40.0, 0.2 * n - 40.0, n)[::direction].copy()
            rows = ramp[:, None, None] * np.ones((1, hkv, d)) / (2.0 * d ** 0.5) + 0.05 * rng.standard_normal((n, hkv, d))
            for j in range(n):
                kc[tables[b][j // bs] * bs + j % bs] = torch.from_numpy(rows[j].astype(np.float32))
        kc = kc.to(torch.bfloat16)
        # (with a window the kernels also start rows whose first subtiles hold no visible key, far below zero)
        for window in (0, 100):
            want = po.paged_prefill_chunk(q, kc, vc, tables, prefix, chunk, bs, d ** -0.5, window=window)
            out = torch.zeros(len(chunk) * cmax, hq, d, device=DEV, dtype=torch.bfloat16)
            ops.prefill_paged(q.reshape(-1, hq, d).to(DEV), kc.to(DEV), vc.to(DEV), tables_to_device(tables),
                              _i32([p + c for p, c in zip(prefix, chunk)]), _i32(chunk),
                              _i32(np.arange(len(chunk)) * cmax), cmax, bs, d ** -0.5, out=out, window=window)
            assert_close(out.reshape(len(chunk), cmax, hq, d), want, 2e-2,
                         f"logits {'rising' if direction > 0 else 'falling'}, window {window}")


@pytest.mark.parametrize("d,dtype,tol", [(80, torch.bfloat16, 2e-2), (96, torch.float16, 2e-2), (192, torch.bfloat16, 2e-2),
                                         (40, torch.float32, 1e-5), (112, torch.float32, 1e-5)])
def test_chunked_prefill_other_head_sizes(d, dtype, tol):
    """Head sizes between the compiled ones (multiples of 8 up to 256) take the next larger size's kernel (the
    vector kernel above 128 and for fp32): chunked prefill over a shared prefix, windows included."""
    announce(f"chunked prefill head_dim {d} {dtype}")
    w = make_prefill_c3(num_seqs=3, prefix_len=64, chunk_len=37, num_q_heads=6, num_kv_heads=2, head_dim=d, dtype=dtype)
    got, kc, vc = _run_chunked(w)
    want = po.paged_prefill_chunk(w.q, kc.cpu(), vc.cpu(), w.block_tables, [64] * 3, [37] * 3, w.block_size, w.scale)
    assert_close(got, want, tol, f"head_dim {d}")
    S, C = w.num_seqs, w.chunk_len
    win = ops.prefill_paged(w.q.reshape(S * C, 6, d).to(DEV), kc, vc, tables_to_device(w.block_tables),
                            _i32([64 + C] * S), _i32([C] * S), _i32(np.arange(S) * C), C, w.block_size, w.scale, window=20)
    want = po.paged_prefill_chunk(w.q, kc.cpu(), vc.cpu(), w.block_tables, [64] * 3, [37] * 3, w.block_size, w.scale,
                                  window=20)
    assert_close(win.reshape(S, C, 6, d), want, tol, f"head_dim {d}, window 20")


@pytest.mark.parametrize("d,dtype", [(96, torch.bfloat16), (72, torch.float16), (120, torch.bfloat16), (104, torch.float16),
                                     (48, torch.bfloat16), (40, torch.float16), (56, torch.bfloat16),
                                     (24, torch.bfloat16), (8, torch.float16), (16, torch.bfloat16),
                                     (160, torch.bfloat16), (192, torch.float16), (248, torch.bfloat16), (136, torch.float16)])
def test_head_sizes_between_the_compiled_ones_on_the_matrix_cores(d, dtype):
    """The reference takes any head_dim (attention/config.py:22-24).  Multiples of 8 up to 256 run the matrix-core
    kernel of the next larger head size (rows in memory keep their size; the 16-byte chunks past a row's end are
    zeros in Q^T and are never stored): dense rows of any length as one block per sequence (several groups per
    workgroup, the group at the end of the pool), with packed documents and a window, and chunked prefill over a
    shared prefix with ragged chunks - against the checker and against the vector kernel on the same inputs."""
    announce(f"prefill on the matrix cores, head_dim {d} {dtype}")
    rng = np.random.default_rng(d)
    hq, hkv = 8, 2
    for b, t, doc_lens in ((2, 333, (40, 200, 93)), (3, 6, (2, 4)), (1, 130, (130,))):
        q, k, v = (torch.from_numpy(rng.standard_normal((b, t, h, d)).astype(np.float32)).to(dtype) for h in (hq, hkv, hkv))
        ident = torch.arange(b, dtype=torch.int32, device=DEV).reshape(b, 1).contiguous()
        lens = _i32([t] * b)
        bounds = np.asarray(po.document_boundaries(doc_lens))
        first = bounds[np.searchsorted(bounds[1:], np.arange(t), side="right")].astype(np.int32)
        first = torch.from_numpy(np.tile(first, b)).to(DEV)
        for docs, window in ((None, 0), (doc_lens, 0), (None, 40), (doc_lens, 40)):
            args = (q.reshape(b * t, hq, d).to(DEV), k.reshape(b * t, hkv, d).to(DEV), v.reshape(b * t, hkv, d).to(DEV),
                    ident, lens, lens, _i32(np.arange(b) * t), t, t, d ** -0.5)
            # the output starts as a pattern: chunks past a row's end must not be stored anywhere
            out = torch.full((b * t + 1, hq, d), 7.0, dtype=dtype, device=DEV)
            got = ops.prefill_paged(*args, out=out[: b * t], window=window, row_first_key=first if docs else None)
            assert (out[b * t] == 7.0).all(), "a store past the last row"
            vec = ops.prefill_paged(*args, window=window, row_first_key=first if docs else None, rowwise=True)
            want = po.dense_prefill(q, k, v, d ** -0.5, window=window, doc_lens=docs)
            assert_close(got.reshape(b, t, hq, d), want, 2e-2, f"{b} x {t}, documents {docs}, window {window}")
            assert_close(got.reshape(b, t, hq, d), vec.reshape(b, t, hq, d).cpu(), 2e-2, f"{b} x {t} against the vector kernel")
    # chunked prefill over a shared prefix, ragged chunks and prefixes, 16-token blocks in random order
    w = make_prefill_c3(num_seqs=3, prefix_len=208, chunk_len=77, num_q_heads=6, num_kv_heads=2, head_dim=d, dtype=dtype)
    got, kc, vc = _run_chunked(w)
    want = po.paged_prefill_chunk(w.q, kc.cpu(), vc.cpu(), w.block_tables, [208] * 3, [77] * 3, w.block_size, w.scale)
    assert_close(got, want, 2e-2, f"chunked, head_dim {d}")
    S, C = w.num_seqs, w.chunk_len
    ctx, ql = [208 + 77, 208 + 30, 100 + 5], [77, 30, 5]
    out = ops.prefill_paged(w.q.reshape(S * C, 6, d).to(DEV), kc, vc, tables_to_device(w.block_tables), _i32(ctx), _i32(ql),
                            _i32(np.arange(S) * C), C, w.block_size, w.scale).reshape(S, C, 6, d)
    want = po.paged_prefill_chunk(w.q, kc.cpu(), vc.cpu(), w.block_tables, [c - n for c, n in zip(ctx, ql)], ql,
                                  w.block_size, w.scale)
    for s_, n in enumerate(ql):
        assert_close(out[s_, :n], want[s_, :n], 2e-2, f"ragged chunk {s_}, head_dim {d}")
