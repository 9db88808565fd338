"""Arbitrary mask predicates (``ctx.block_mask`` objects other than the structured PagedMask): pa_attend_masked
against the checker's dense statement, and through the backend in the three places the reference hands a
block mask to flex_attention (flex_backend.py:170-178 dense prefill, :220-225 decode) plus chunked prefill."""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import ops
from research_amd.inference import CacheConfig, HipPagedAttentionBackend, InferenceContext
from research_amd.inference.attention.mask import create_attention_mask
from tests.gpu_helpers import DEV, announce, assert_close, tables_to_device

pytestmark = pytest.mark.gpu


def _i32(x):
    return torch.tensor(list(x), dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2), (torch.float16, 5e-3)])
@pytest.mark.parametrize("d,hq,hkv", [(128, 8, 2), (64, 4, 4), (256, 2, 1), (40, 6, 3)])
def test_attend_masked_against_the_checker(dtype, tol, d, hq, hkv):
    """Random masks per head and shared by the heads, rows that keep nothing, kept keys past the context end (zero
    rows), an absent block, ragged q rows, a key count that is not a multiple of 32."""
    announce(f"masked attention {dtype} d={d} hq={hq} hkv={hkv}")
    rng = np.random.default_rng(5 + d)
    bs, nb = 8, 24
    ctx, ql = [70, 33, 9], [5, 3, 4]
    n_keys, tmax = 77, 5
    perm = rng.permutation(nb)
    tables = [perm[:9].tolist(), perm[9:14].tolist(), perm[14:16].tolist()]
    tables[0][3] = -1  # an absent block inside the context
    kc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
    vc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
    q = torch.from_numpy(rng.standard_normal((3, tmax, hq, d)).astype(np.float32)).to(dtype)
    width = max(len(t) for t in tables)
    dev_tables = torch.tensor([t + [-1] * (width - len(t)) for t in tables], dtype=torch.int32, device=DEV)
    for heads in (hq, 1):
        keep = rng.random((3, tmax, heads, n_keys)) < 0.4
        keep[0, 2] = False
        keep[2, 1, :, 9:] = True
        want = po.paged_attend_masked(q, kc, vc, tables, ctx, ql, keep, bs, d ** -0.5)
        words = ops.pack_mask(torch.from_numpy(keep.reshape(3 * tmax, heads, n_keys)).to(DEV))
        out = torch.full((3 * tmax, hq, d), 7.0, dtype=dtype, device=DEV)
        ops.attend_masked(q.reshape(-1, hq, d).to(DEV), kc.to(DEV), vc.to(DEV), dev_tables, _i32(ctx), _i32(ql),
                          _i32(np.arange(3) * tmax), tmax, bs, d ** -0.5, words, n_keys, out=out)
        got = out.reshape(3, tmax, hq, d)
        for b in range(3):
            assert_close(got[b, : ql[b]], want[b, : ql[b]], tol, f"mask heads {heads} sequence {b}")
            assert (got[b, ql[b]:] == 7.0).all()  # rows past q_lens are not written


def _backend(dtype=torch.float32, bs=8, nb=16, hkv=2, d=64):
    be = HipPagedAttentionBackend(CacheConfig(num_layers=1, num_kv_heads=hkv, head_dim=d, num_blocks=nb, block_size=bs,
                                              dtype=dtype, device="cuda"))
    be.set_num_heads(4)
    return be


def test_predicates_through_the_backend():
    announce("mask predicates through the backend")
    rng = np.random.default_rng(9)
    be = _backend()
    B, T, H, D = 2, 21, 4, 64
    q = torch.from_numpy(rng.standard_normal((B, T, H, D)).astype(np.float32))
    k = torch.from_numpy(rng.standard_normal((B, T, 2, D)).astype(np.float32))
    v = torch.from_numpy(rng.standard_normal((B, T, 2, D)).astype(np.float32))
    dense = lambda keep: po.paged_attend_masked(q, k.reshape(B * T, 2, D), v.reshape(B * T, 2, D), [[0], [1]], [T, T],
                                                [T, T], keep, T, be.scale)
    qi, ki = np.arange(T)[:, None], np.arange(T)[None, :]

    # (1) dense prefill: a prefix-LM predicate (everything sees the first 5 keys, the rest is causal)
    prefix_lm = lambda b, h, q_idx, kv_idx: (kv_idx < 5) | (q_idx >= kv_idx)
    out = be.forward(q.cuda(), k.cuda(), v.cuda(), 0, InferenceContext(is_prefill=True, block_mask=prefix_lm))
    keep = np.broadcast_to(((ki < 5) | (qi >= ki))[None, :, None, :], (B, T, 1, T))
    assert_close(out, dense(keep), 1e-5, "prefix-LM predicate, dense prefill")

    # (2) a predicate that depends on the head and the sequence (each head its own window, sequence 1 one more)
    per_head = lambda b, h, q_idx, kv_idx: (q_idx >= kv_idx) & (q_idx - kv_idx <= h + b)
    out = be.forward(q.cuda(), k.cuda(), v.cuda(), 0, InferenceContext(is_prefill=True, block_mask=per_head))
    keep = np.stack([np.stack([(qi >= ki) & (qi - ki <= h + b) for h in range(H)], 1) for b in range(B)])
    assert_close(out, dense(keep), 1e-5, "per-head windows")
    # the same predicate evaluated a few query rows at a time (what bounds the memory of long steps)
    small = _backend()
    small._mask_round_elems = B * H * T * 4  # four rows per round: six rounds
    out = small.forward(q.cuda(), k.cuda(), v.cuda(), 0, InferenceContext(is_prefill=True, block_mask=per_head))
    assert_close(out, dense(keep), 1e-5, "per-head windows, evaluated in rounds of rows")

    # (3) the causal predicate and the reference's own mask object give the causal kernels' result
    causal = be.forward(q.cuda(), k.cuda(), v.cuda(), 0, InferenceContext(is_prefill=True))
    out = be.forward(q.cuda(), k.cuda(), v.cuda(), 0,
                     InferenceContext(is_prefill=True, block_mask=lambda b, h, q_idx, kv_idx: q_idx >= kv_idx))
    assert_close(out, causal.float().cpu().numpy(), 1e-5, "causal predicate")
    try:
        from torch.nn.attention.flex_attention import create_block_mask
        block_mask = create_block_mask(lambda b, h, q_idx, kv_idx: (q_idx >= kv_idx) & (q_idx - kv_idx < 6), B, None, T, T,
                                       device="cuda")
    except Exception as exc:  # this torch build cannot build block masks on the device: the callables above cover it
        block_mask = None
        print("create_block_mask unavailable:", type(exc).__name__)
    if block_mask is not None:
        out = be.forward(q.cuda(), k.cuda(), v.cuda(), 0, InferenceContext(is_prefill=True, block_mask=block_mask))
        windowed = be.forward(q.cuda(), k.cuda(), v.cuda(), 0, InferenceContext(
            is_prefill=True, block_mask=create_attention_mask(batch_size=B, seq_len=T, sliding_window=6, block_size=8,
                                                              device="cuda")))
        assert_close(out, windowed.float().cpu().numpy(), 1e-5, "a FlexAttention BlockMask object")

    # (4) chunked prefill over the cache: q_idx is the row's position in the sequence
    be.clear_cache()
    ctx_lens, pre = [T, 13], [T - 6, 13 - 6]
    tables = ((3, 1, 6), (7, 2))
    for b in range(B):
        slots = [tables[b][p // 8] * 8 + p % 8 for p in range(ctx_lens[b])]
        be._store_kv(k[b, : ctx_lens[b]].cuda(), v[b, : ctx_lens[b]].cuda(), 0, tuple(slots))
    window = lambda b, h, q_idx, kv_idx: (q_idx >= kv_idx) & (q_idx - kv_idx < 4)
    qc = q[:, :6]
    ctx = InferenceContext(is_prefill=True, block_tables=tables, seq_lens=tuple(ctx_lens), prefix_lens=tuple(pre),
                           block_mask=window)
    out = be.forward(qc.cuda(), None, None, 0, ctx)
    want = po.paged_prefill_chunk(qc, be.k_cache[0].cpu(), be.v_cache[0].cpu(), tables, pre, [6, 6], 8, be.scale, window=4)
    assert_close(out, want, 1e-5, "sliding-window predicate over a cached prefix")

    # (5) decode, literally as the reference: q_idx = 0, kv_idx over the longest sequence, zero rows past a
    # shorter sequence's end take part where the predicate keeps them
    keep_first = lambda b, h, q_idx, kv_idx: kv_idx < 17
    ctx = InferenceContext(is_prefill=False, block_tables=tables, seq_lens=tuple(ctx_lens), block_mask=keep_first)
    q1 = q[:, :1]
    out = be.forward(q1.cuda(), None, None, 0, ctx)
    keep = np.broadcast_to((np.arange(T) < 17)[None, None, None, :], (B, 1, 1, T))
    want = po.paged_attend_masked(q1, be.k_cache[0].cpu(), be.v_cache[0].cpu(), tables, ctx_lens, [1, 1], keep, 8, be.scale)
    assert_close(out, want, 1e-5, "decode under a predicate")
    lit = po.decode_literal(q1[:1], be.k_cache[0].cpu(), be.v_cache[0].cpu(), tables[:1], (17,), 8, be.scale)
    assert_close(out[:1], lit, 1e-5, "the first sequence: plain decode over its first 17 keys")
    with pytest.raises(NotImplementedError):
        be.forward(q1.cuda(), None, None, 0, InferenceContext(is_prefill=False, block_tables=tables,
                                                             seq_lens=tuple(ctx_lens), block_mask=object()))


def test_predicates_over_an_fp8_pool():
    """A mask predicate with ``kv_format="fp8_e4m3"``: the masked kernel widens the pool's bytes with the tile's
    scale; against the checker on the dequantised pool (6e-2), in chunked prefill and in decode."""
    announce("mask predicates over an fp8 pool")
    rng = np.random.default_rng(4)
    bs, nb, hkv, hq, d = 16, 12, 2, 4, 64
    be = HipPagedAttentionBackend(CacheConfig(num_layers=1, num_kv_heads=hkv, head_dim=d, num_blocks=nb, block_size=bs,
                                              dtype=torch.bfloat16, device="cuda", kv_format="fp8_e4m3"))
    be.set_num_heads(hq)
    kp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16)
    vp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16)
    be.quantize_from(kp.cuda(), vp.cuda(), 0)
    kd = po.dequantize_kv_e4m3(be.k_cache[0].cpu().view(torch.uint8), be.k_scale[0].cpu(), bs)
    vd = po.dequantize_kv_e4m3(be.v_cache[0].cpu().view(torch.uint8), be.v_scale[0].cpu(), bs)
    tables, ctx_lens, pre = ((3, 1, 6, 9), (7, 2, 5)), [60, 41], [52, 33]
    q = torch.from_numpy(rng.standard_normal((2, 8, hq, d)).astype(np.float32)).to(torch.bfloat16)
    window = lambda b, h, q_idx, kv_idx: (q_idx >= kv_idx) & (q_idx - kv_idx < 11 + h)
    ctx = InferenceContext(is_prefill=True, block_tables=tables, seq_lens=tuple(ctx_lens), prefix_lens=tuple(pre),
                           block_mask=window)
    out = be.forward(q.cuda(), None, None, 0, ctx)
    qi = (np.asarray(pre)[:, None] + np.arange(8)[None, :])[:, :, None, None]
    ki = np.arange(60)[None, None, None, :]
    hi = np.arange(hq)[None, None, :, None]
    keep = (qi >= ki) & (qi - ki < 11 + hi)
    want = po.paged_attend_masked(q, kd, vd, tables, ctx_lens, [8, 8], keep, bs, be.scale)
    assert_close(out, want, 6e-2, "per-head windows over an fp8 pool, chunked prefill")
    q1 = q[:, :1]
    first = lambda b, h, q_idx, kv_idx: kv_idx < 37
    out = be.forward(q1.cuda(), None, None, 0, InferenceContext(is_prefill=False, block_tables=tables,
                                                               seq_lens=tuple(ctx_lens), block_mask=first))
    keep = np.broadcast_to((np.arange(60) < 37)[None, None, None, :], (2, 1, 1, 60))
    want = po.paged_attend_masked(q1, kd, vd, tables, ctx_lens, [1, 1], keep, bs, be.scale)
    assert_close(out, want, 6e-2, "decode under a predicate over an fp8 pool")
