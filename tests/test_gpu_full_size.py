"""The benchmark workloads (research_amd/workloads.py) at full size on the GPU.

Decode (c4, c5): EVERY sequence against the CPU checker with the real queries,
in groups of sequences on a compacted copy of their blocks (block ids do not
matter, a property the checker itself is pinned on; a group keeps the float64
copies the checker makes small), plus a size-independent property over the
whole batch (with q = 0 attention is uniform, so each output row is the mean
of the sequence's V rows, computed here with plain torch indexing).  Prefill
(c3): all 32 sequences against the checker, and the two kernels against each
other on every output.
"""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import ops
from research_amd.workloads import make_decode, make_prefill_c3
from tests.gpu_helpers import DEV, announce, assert_close, tables_to_device

pytestmark = pytest.mark.gpu


def _compact(w, seqs, k_pool, v_pool):
    """Pools holding only the blocks of `seqs`, renumbered 0.., and the matching tables."""
    bs = w.block_size
    blocks = np.concatenate([np.asarray(w.block_tables[b]) for b in seqs])
    slots = torch.from_numpy((blocks[:, None] * bs + np.arange(bs)[None, :]).reshape(-1))
    tables, at = [], 0
    for b in seqs:
        n = len(w.block_tables[b])
        tables.append(list(range(at, at + n)))
        at += n
    return k_pool[slots], v_pool[slots], tables


def _mean_of_v_rows(w, v_pool_dev, dequant=None):
    """float32 [B, Hkv, D]: mean over each sequence's V rows, by torch indexing on the device."""
    bs = w.block_size
    out = torch.zeros(w.batch, w.num_kv_heads, w.head_dim, dtype=torch.float32, device=DEV)
    for b in range(w.batch):
        n = int(w.seq_lens[b])
        if n == 0:
            continue
        blocks = torch.from_numpy(np.asarray(w.block_tables[b], dtype=np.int64)).to(DEV)
        pos = torch.arange(n, device=DEV)
        blk = blocks[pos // bs]
        rows = v_pool_dev[blk * bs + pos % bs].float()
        if dequant is not None:
            rows = rows * dequant[blk][:, :, None]
        out[b] = rows.mean(0)
    return out


def _assert_mean(got, want, rel, floor, what):
    """|got - want| <= rel*|want| + floor: `rel` is the rounding of the 16-bit output, `floor` what a sum of
    thousands of fp32 terms may lose; a dropped or doubled 16-key block of a 2000-key sequence moves the mean
    of N(0,1) rows by about 2e-3."""
    got, want = got.double().cpu().numpy(), want.double().cpu().numpy()
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    excess = np.abs(got - want) - rel * np.abs(want)
    assert excess.max() <= floor, f"{what}: {excess.max():.3e} over the bar at {np.unravel_index(excess.argmax(), excess.shape)}"


def test_c4_full_size():
    """workload c4: B=256, 840 539 keys in 52 656 blocks, bf16."""
    announce("decode c4 full size")
    w = make_decode("c4")
    assert w.batch == 256 and w.total_tokens == 840539
    q, kp, vp = w.q.to(DEV), w.k_pool.to(DEV), w.v_pool.to(DEV)
    tables = tables_to_device(w.block_tables)
    lens = torch.from_numpy(w.seq_lens.astype(np.int32)).to(DEV)
    ws = ops.decode_workspace(q, kp)
    got = ops.decode(q, kp, vp, tables, lens, w.block_size, w.scale, ws).float().cpu()
    # the checker on every sequence, 16 at a time
    for g0 in range(0, w.batch, 16):
        seqs = list(range(g0, min(w.batch, g0 + 16)))
        kc, vc, tc = _compact(w, seqs, w.k_pool, w.v_pool)
        want = po.paged_decode(w.q[seqs], kc, vc, tc, w.seq_lens[seqs], w.block_size, w.scale)
        assert_close(got[seqs], want, 2e-2, f"c4 sequences {g0}..{seqs[-1]} against the checker")
    # every sequence: uniform attention = mean of its V rows
    uni = ops.decode(torch.zeros_like(q), kp, vp, tables, lens, w.block_size, w.scale, ws).float()
    mean = _mean_of_v_rows(w, vp).repeat_interleave(w.num_q_heads // w.num_kv_heads, dim=1)
    _assert_mean(uni, mean, 2.0 ** -8, 2e-4, "c4 uniform attention over all 256 sequences")
    # the same launch again gives the same bits (no dependence on workspace contents or timing)
    again = ops.decode(q, kp, vp, tables, lens, w.block_size, w.scale, ws).float().cpu()
    assert torch.equal(got, again)


def test_c5_full_size_fp8():
    """workload c5: B=8, 802 997 keys, fp8-e4m3 pool with per-(block, kv head) scales."""
    announce("decode c5 full size")
    w = make_decode("c5")
    assert w.batch == 8 and w.total_tokens == 802997
    q = w.q.to(DEV)
    k8, ks = ops.quantize_kv_e4m3(w.k_pool.to(DEV), w.block_size)
    v8, vs = ops.quantize_kv_e4m3(w.v_pool.to(DEV), w.block_size)
    tables = tables_to_device(w.block_tables)
    lens = torch.from_numpy(w.seq_lens.astype(np.int32)).to(DEV)
    ws = ops.decode_workspace(q, k8)
    got = ops.decode(q, k8, v8, tables, lens, w.block_size, w.scale, ws, k_scale=ks, v_scale=vs).float().cpu()
    # the checker (dequantise, then attend) on every sequence, two at a time
    bs = w.block_size
    k8c, v8c, ksc, vsc = k8.cpu().view(torch.uint8), v8.cpu().view(torch.uint8), ks.cpu(), vs.cpu()
    for g0 in range(0, w.batch, 2):
        seqs = [g0, g0 + 1]
        kq, vq, tc = _compact(w, seqs, k8c, v8c)
        blocks = np.concatenate([np.asarray(w.block_tables[b]) for b in seqs])
        kd = po.dequantize_kv_e4m3(kq, ksc[blocks], bs)
        vd = po.dequantize_kv_e4m3(vq, vsc[blocks], bs)
        want = po.paged_decode(w.q[seqs], kd, vd, tc, w.seq_lens[seqs], bs, w.scale)
        assert_close(got[seqs], want, 6e-2, f"c5 sequences {seqs} against the checker")
    uni = ops.decode(torch.zeros_like(q), k8, v8, tables, lens, bs, w.scale, ws, k_scale=ks, v_scale=vs).float()
    mean = _mean_of_v_rows(w, v8, dequant=vs).repeat_interleave(w.num_q_heads // w.num_kv_heads, dim=1)
    # (the kernel rounds p * v_scale to the 16-bit query type once per block: 2^-9 relative, same sign per block)
    _assert_mean(uni, mean, 2.0 ** -7, 2e-4, "c5 uniform attention over all 8 sequences")


def test_c3_full_size_two_kernels_and_sample():
    """workload c3: 32 x (2048 shared + 256 own) tokens; matrix-core kernel against the vector kernel on
    every output element, and against the checker on all 32 sequences."""
    announce("prefill c3 full size")
    w = make_prefill_c3()
    S, C, P = w.num_seqs, w.chunk_len, w.prefix_len
    shape = (w.num_blocks * w.block_size, w.num_kv_heads, w.head_dim)
    kc = torch.zeros(shape, dtype=w.dtype, device=DEV)
    vc = torch.zeros_like(kc)
    ops.kv_scatter(kc, vc, w.k_prefix.to(DEV), w.v_prefix.to(DEV), torch.from_numpy(w.prefix_slots()).to(DEV))
    ops.kv_scatter(kc, vc, w.k_chunk.reshape(S * C, *shape[1:]).to(DEV), w.v_chunk.reshape(S * C, *shape[1:]).to(DEV),
                   torch.from_numpy(w.chunk_slots()).to(DEV))
    q = w.q.reshape(S * C, w.num_q_heads, w.head_dim).to(DEV)
    tables = tables_to_device(w.block_tables)
    i32 = lambda x: torch.tensor(list(x), dtype=torch.int32, device=DEV)
    args = (q, kc, vc, tables, i32([P + C] * S), i32([C] * S), i32(np.arange(S) * C), C, w.block_size, w.scale)
    mfma = ops.prefill_paged(*args).float().cpu()
    rowwise = ops.prefill_paged(*args, rowwise=True).float().cpu()
    assert_close(mfma, rowwise, 2e-2, "matrix-core kernel against the vector kernel, all 32 x 256 x 32 rows")
    seqs = list(range(S))
    want = po.paged_prefill_chunk(w.q[seqs], kc.cpu(), vc.cpu(), [w.block_tables[s] for s in seqs], [P] * len(seqs),
                                  [C] * len(seqs), w.block_size, w.scale)
    assert_close(mfma.reshape(S, C, w.num_q_heads, w.head_dim)[seqs], want, 2e-2, "c3 against the checker, all sequences")
