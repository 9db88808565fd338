"""Pins the CPU checker (oracle/paged_oracle.py) before anything is compared with it.

The reference holds no stored tensors for this path; its tests assert a few
integer facts, one store round trip and "prefill equals torch SDPA" within
0.01 / 0.001.  Everything else is pinned here by independent routes: a
pure-Python softmax, the torch library routine the reference itself calls,
closed forms and invariances - each chosen so that a plausible slip (wrong
head mapping, wrong slot arithmetic, off-by-one in the causal offset, dropped
padding term) fails at least one test.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import paged_oracle as po
from research_amd.workloads import make_decode, make_prefill_c3


def _tiny_pool(rng, num_blocks=6, bs=4, hkv=2, d=8):
    k = torch.from_numpy(rng.standard_normal((num_blocks * bs, hkv, d)).astype(np.float32))
    v = torch.from_numpy(rng.standard_normal((num_blocks * bs, hkv, d)).astype(np.float32))
    return k, v


# ---------------------------------------------------------------- scatter / gather
def test_scatter_reference_assertion():
    """slots 0..3 of layer 0 receive rows 0..3 (test_kv_cache.py:101-111 of the reference)."""
    g = torch.Generator().manual_seed(0)
    k = torch.randn(1, 4, 4, 32, generator=g).to(torch.bfloat16)
    v = torch.randn(1, 4, 4, 32, generator=g).to(torch.bfloat16)
    kc = torch.zeros(64, 4, 32, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    po.kv_scatter(kc, vc, k.reshape(-1, 4, 32), v.reshape(-1, 4, 32), tuple(range(4)))
    assert torch.equal(kc[0], k[0, 0]) and torch.equal(vc[3], v[0, 3])
    assert not kc[4:].any()


def test_scatter_skips_negative_and_matches_index_put():
    rng = np.random.default_rng(1)
    src_k, src_v = _tiny_pool(rng, num_blocks=2)
    slots = [5, -1, 0, 17, -1, 9, 2, 23]
    kc, vc = torch.zeros(24, 2, 8), torch.zeros(24, 2, 8)
    po.kv_scatter(kc, vc, src_k, src_v, slots)
    # the reference's statement, with torch indexing (flex_backend.py:136-142)
    st = torch.tensor(slots)
    ek, ev = torch.zeros(24, 2, 8), torch.zeros(24, 2, 8)
    ek[st[st >= 0]] = src_k[st >= 0]
    ev[st[st >= 0]] = src_v[st >= 0]
    assert torch.equal(kc, ek) and torch.equal(vc, ev)


def test_gather_closed_form_and_loop():
    rng = np.random.default_rng(2)
    kc, vc = _tiny_pool(rng)
    tables = [(3, 0, 5), (1,), (4, 2)]
    lens = [10, 3, 8]
    kg, vg = po.kv_gather_padded(kc, vc, tables, lens, 4)
    kl, vl = po.kv_gather_loop(kc, vc, tables, lens, 4)
    assert torch.equal(kg, kl) and torch.equal(vg, vl)
    assert kg.shape == (3, 10, 2, 8)
    assert torch.equal(kg[0, 9], kc[5 * 4 + 1]) and torch.equal(vg[2, 6], vc[2 * 4 + 2])
    assert not kg[1, 3:].any() and not vg[2, 8:].any()


def test_gather_short_table_leaves_zeros():
    rng = np.random.default_rng(3)
    kc, vc = _tiny_pool(rng)
    kg, vg = po.kv_gather_padded(kc, vc, [(2,)], [7], 4)
    kl, _ = po.kv_gather_loop(kc, vc, [(2,)], [7], 4)
    assert torch.equal(kg, kl)
    assert torch.equal(kg[0, :4], kc[8:12]) and not kg[0, 4:].any()


def test_gather_of_scatter_is_identity():
    rng = np.random.default_rng(4)
    bs, tables, lens = 4, [(5, 1, 3), (0, 4)], [11, 6]
    kc, vc = torch.zeros(24, 2, 8), torch.zeros(24, 2, 8)
    rows_k, rows_v = _tiny_pool(rng, num_blocks=5)
    slots = [po.slot_of(t, p, bs) for t, n in zip(tables, lens) for p in range(n)]
    po.kv_scatter(kc, vc, rows_k[:17], rows_v[:17], slots)
    kg, vg = po.kv_gather_padded(kc, vc, tables, lens, bs)
    assert torch.equal(kg[0, :11], rows_k[:11]) and torch.equal(kg[1, :6], rows_k[11:17])
    assert torch.equal(vg[0, :11], rows_v[:11]) and torch.equal(vg[1, :6], rows_v[11:17])


# ---------------------------------------------------------------- decode
def _python_decode(q, kc, vc, tables, lens, bs, scale, n_zero=None):
    """Independent statement: scalar loops and math.exp only."""
    B, Hq, D = q.shape
    Hkv = kc.shape[1]
    n_rep = Hq // Hkv
    out = np.zeros((B, Hq, D))
    for b in range(B):
        for h in range(Hq):
            g = h // n_rep
            logits, vals = [], []
            for pos in range(lens[b]):
                blk = pos // bs
                if blk < len(tables[b]):
                    slot = tables[b][blk] * bs + pos % bs
                    logits.append(scale * sum(float(q[b, h, e]) * float(kc[slot, g, e]) for e in range(D)))
                    vals.append([float(x) for x in vc[slot, g]])
                else:
                    logits.append(0.0)
                    vals.append([0.0] * D)
            for _ in range(0 if n_zero is None else n_zero[b]):
                logits.append(0.0)
                vals.append([0.0] * D)
            m = max(logits)
            w = [math.exp(x - m) for x in logits]
            den = sum(w)
            for e in range(D):
                out[b, h, e] = sum(wi * vi[e] for wi, vi in zip(w, vals)) / den
    return out


def test_decode_against_python_loops():
    rng = np.random.default_rng(5)
    kc, vc = _tiny_pool(rng)
    q = torch.from_numpy(rng.standard_normal((3, 4, 8)).astype(np.float32))
    tables, lens = [(3, 0, 5), (1,), (4, 2)], [10, 3, 8]
    got = po.paged_decode(q, kc, vc, tables, lens, 4, 0.35)
    want = _python_decode(q.numpy(), kc.numpy(), vc.numpy(), tables, lens, 4, 0.35)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


def test_decode_short_table_counts_zero_keys():
    rng = np.random.default_rng(6)
    kc, vc = _tiny_pool(rng)
    q = torch.from_numpy(rng.standard_normal((1, 2, 8)).astype(np.float32))
    got = po.paged_decode(q, kc, vc, [(2,)], [7], 4, 0.5)
    want = _python_decode(q.numpy(), kc.numpy(), vc.numpy(), [(2,)], [7], 4, 0.5)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
    # and the reference's own composition (gather zeros, attend everything) agrees
    lit = po.decode_literal(q[:, None], kc, vc, [(2,)], [7], 4, 0.5)[:, 0]
    np.testing.assert_allclose(got, lit.numpy(), rtol=2e-6, atol=2e-6)


def test_decode_equals_sdpa_on_gathered_when_lengths_equal():
    rng = np.random.default_rng(7)
    kc, vc = _tiny_pool(rng, num_blocks=8)
    q = torch.from_numpy(rng.standard_normal((2, 4, 8)).astype(np.float32))
    tables, lens = [(6, 1, 7), (0, 3, 2)], [9, 9]
    got = po.paged_decode(q, kc, vc, tables, lens, 4, 8**-0.5)
    lit = po.decode_literal(q[:, None], kc, vc, tables, lens, 4, 8**-0.5)[:, 0]
    np.testing.assert_allclose(got, lit.numpy(), rtol=2e-6, atol=2e-6)


def test_decode_gqa_mapping_against_expanded_heads():
    """q head h must read kv head h // n_rep (not h % Hkv)."""
    rng = np.random.default_rng(8)
    kc, vc = _tiny_pool(rng, hkv=2)
    q = torch.from_numpy(rng.standard_normal((1, 6, 8)).astype(np.float32))
    tables, lens = [(3, 0, 5)], [12]
    got = po.paged_decode(q, kc, vc, tables, lens, 4, 0.3)
    kx, vx = kc.repeat_interleave(3, dim=1), vc.repeat_interleave(3, dim=1)  # MHA with 6 kv heads
    want = po.paged_decode(q, kx, vx, tables, lens, 4, 0.3)
    np.testing.assert_allclose(got, want, rtol=1e-12)
    wrong = po.paged_decode(q, torch.cat([kc] * 3, dim=1), torch.cat([vc] * 3, dim=1), tables, lens, 4, 0.3)
    assert np.abs(got - wrong).max() > 1e-3


def test_decode_invariant_under_pool_permutation():
    rng = np.random.default_rng(9)
    bs, nb = 4, 6
    kc, vc = _tiny_pool(rng, num_blocks=nb, bs=bs)
    q = torch.from_numpy(rng.standard_normal((2, 4, 8)).astype(np.float32))
    tables, lens = [(3, 0, 5), (4, 2)], [10, 7]
    base = po.paged_decode(q, kc, vc, tables, lens, bs, 0.4)
    perm = rng.permutation(nb)  # new id of block i is perm[i]
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    for old in range(nb):
        kc2[perm[old] * bs : (perm[old] + 1) * bs] = kc[old * bs : (old + 1) * bs]
        vc2[perm[old] * bs : (perm[old] + 1) * bs] = vc[old * bs : (old + 1) * bs]
    tables2 = [tuple(int(perm[b]) for b in t) for t in tables]
    np.testing.assert_allclose(po.paged_decode(q, kc2, vc2, tables2, lens, bs, 0.4), base, rtol=1e-12)


def test_decode_constant_value_rows():
    rng = np.random.default_rng(10)
    kc, vc = _tiny_pool(rng)
    vc[:] = torch.tensor([1.5, -2.0, 0.25, 3.0, 0.0, 1.0, -1.0, 7.0])
    q = torch.from_numpy(rng.standard_normal((1, 4, 8)).astype(np.float32))
    out = po.paged_decode(q, kc, vc, [(0, 1, 2)], [11], 4, 1.0)
    np.testing.assert_allclose(out, np.broadcast_to(vc[0, 0].numpy(), out.shape), rtol=1e-12)


def test_pad_zero_keys_closed_form_and_literal():
    """Ragged batch: the reference's zero padding adds (Lmax-L) e^{-m} to the denominator."""
    rng = np.random.default_rng(11)
    kc, vc = _tiny_pool(rng)
    q = torch.from_numpy(rng.standard_normal((3, 4, 8)).astype(np.float32))
    tables, lens, bs, scale = [(3, 0, 5), (1,), (4, 2)], [10, 3, 8], 4, 0.35
    got = po.paged_decode(q, kc, vc, tables, lens, bs, scale, pad_zero_keys=True)
    want = _python_decode(q.numpy(), kc.numpy(), vc.numpy(), tables, lens, bs, scale,
                          n_zero=[max(lens) - n for n in lens])
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
    lit = po.decode_literal(q[:, None], kc, vc, tables, lens, bs, scale)[:, 0]
    np.testing.assert_allclose(got, lit.numpy(), rtol=2e-6, atol=2e-6)
    masked = po.paged_decode(q, kc, vc, tables, lens, bs, scale)
    assert np.abs(masked[1] - got[1]).max() > 1e-3  # the two semantics do differ on short rows
    np.testing.assert_allclose(masked[0], got[0], rtol=1e-12)  # and agree on the longest one


def test_per_sequence_baseline_equals_masked_decode():
    w = make_decode("c1")
    tables = [t.tolist() for t in w.block_tables]
    got = po.decode_per_sequence(w.q[:, None], w.k_pool, w.v_pool, tables, w.seq_lens, w.block_size, w.scale)[:, 0]
    want = po.paged_decode(w.q, w.k_pool, w.v_pool, tables, w.seq_lens, w.block_size, w.scale)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-5, atol=1e-5)


def test_c1_both_modes_against_literal():
    w = make_decode("c1")
    assert w.seq_lens.tolist() == [232, 157, 210, 5] and w.num_blocks == 128
    tables = [t.tolist() for t in w.block_tables]
    lit = po.decode_literal(w.q[:, None], w.k_pool, w.v_pool, tables, w.seq_lens, w.block_size, w.scale,
                            vectorised_gather=True)[:, 0].numpy()
    pad = po.paged_decode(w.q, w.k_pool, w.v_pool, tables, w.seq_lens, w.block_size, w.scale, pad_zero_keys=True)
    np.testing.assert_allclose(pad, lit, rtol=1e-5, atol=1e-5)
    masked = po.paged_decode(w.q, w.k_pool, w.v_pool, tables, w.seq_lens, w.block_size, w.scale)
    np.testing.assert_allclose(masked[0], lit[0], rtol=1e-5, atol=1e-5)  # longest sequence: no padding
    assert np.abs(masked[3] - lit[3]).max() > 1e-2  # 5 keys vs 5 keys + 227 zero keys


# ---------------------------------------------------------------- prefill
def test_dense_prefill_reference_recipe():
    """The reference's correctness test (test_kv_cache.py:276-345): B=2,T=8,Hq=4,Hkv=2,D=32, bf16, seed 42."""
    torch.manual_seed(42)
    q = torch.randn(2, 8, 4, 32).to(torch.bfloat16)
    k = torch.randn(2, 8, 2, 32).to(torch.bfloat16)
    v = torch.randn(2, 8, 2, 32).to(torch.bfloat16)
    ref = F.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2).repeat_interleave(2, dim=1),
        v.transpose(1, 2).repeat_interleave(2, dim=1), is_causal=True).transpose(1, 2)
    got = po.dense_prefill(q, k, v, 32**-0.5)
    diff = np.abs(got - ref.to(torch.float64).numpy())
    assert diff.max() < 0.01 and diff.mean() < 0.001  # the reference's own bars (:341-342)
    lit = po.prefill_literal(q.float(), k.float(), v.float(), 32**-0.5)
    np.testing.assert_allclose(got, lit.numpy(), rtol=1e-5, atol=1e-5)


def test_dense_prefill_first_and_last_rows():
    rng = np.random.default_rng(12)
    q = rng.standard_normal((1, 5, 2, 8))
    k = rng.standard_normal((1, 5, 1, 8))
    v = rng.standard_normal((1, 5, 1, 8))
    out = po.dense_prefill(q, k, v, 0.3)
    np.testing.assert_allclose(out[0, 0], np.broadcast_to(v[0, 0, 0], (2, 8)), rtol=1e-12)  # row 0 sees key 0 only
    full = F.scaled_dot_product_attention(
        torch.from_numpy(q[:, 4:5]).transpose(1, 2), torch.from_numpy(k).transpose(1, 2).repeat_interleave(2, 1),
        torch.from_numpy(v).transpose(1, 2).repeat_interleave(2, 1), scale=0.3).transpose(1, 2)
    np.testing.assert_allclose(out[0, 4], full[0, 0].numpy(), rtol=1e-10)  # last row sees everything


def _c3_small(**kw):
    w = make_prefill_c3(num_seqs=3, prefix_len=32, chunk_len=10, num_q_heads=4, num_kv_heads=2, head_dim=16,
                        dtype=torch.float32, **kw)
    kc = torch.zeros(w.num_blocks * w.block_size, 2, 16)
    vc = torch.zeros_like(kc)
    po.kv_scatter(kc, vc, w.k_prefix, w.v_prefix, w.prefix_slots())
    po.kv_scatter(kc, vc, w.k_chunk.reshape(-1, 2, 16), w.v_chunk.reshape(-1, 2, 16), w.chunk_slots())
    return w, kc, vc


def test_chunked_prefill_equals_rows_of_full_causal():
    w, kc, vc = _c3_small()
    S, P, C = w.num_seqs, w.prefix_len, w.chunk_len
    got = po.paged_prefill_chunk(w.q, kc, vc, w.block_tables, [P] * S, [C] * S, w.block_size, w.scale)
    for s in range(S):
        k_full = torch.cat([w.k_prefix, w.k_chunk[s]])[None]
        v_full = torch.cat([w.v_prefix, w.v_chunk[s]])[None]
        q_full = torch.cat([torch.zeros(P, 4, 16), w.q[s]])[None]
        full = po.dense_prefill(q_full, k_full, v_full, w.scale)
        np.testing.assert_allclose(got[s], full[0, P:], rtol=1e-10, atol=1e-12)
        # off-by-one guard: top-left alignment (what is_causal=True would do for q_len < kv_len) differs
        lit = po.prefill_literal(q_full.double(), k_full.double(), v_full.double(), w.scale)
        np.testing.assert_allclose(got[s], lit[0, P:].numpy(), rtol=1e-9, atol=1e-11)


def test_chunked_prefill_without_prefix_is_dense_prefill():
    w = make_prefill_c3(num_seqs=2, prefix_len=0, chunk_len=21, num_q_heads=4, num_kv_heads=2, head_dim=16,
                        dtype=torch.float32)
    kc = torch.zeros(w.num_blocks * w.block_size, 2, 16)
    vc = torch.zeros_like(kc)
    po.kv_scatter(kc, vc, w.k_chunk.reshape(-1, 2, 16), w.v_chunk.reshape(-1, 2, 16), w.chunk_slots())
    got = po.paged_prefill_chunk(w.q, kc, vc, w.block_tables, [0, 0], [21, 21], w.block_size, w.scale)
    np.testing.assert_allclose(got, po.dense_prefill(w.q, w.k_chunk, w.v_chunk, w.scale), rtol=1e-12)


def test_shared_prefix_blocks_equal_private_copies():
    w, kc, vc = _c3_small()
    S, P, C, bs = w.num_seqs, w.prefix_len, w.chunk_len, w.block_size
    assert all(np.array_equal(t[: P // bs], w.block_tables[0][: P // bs]) for t in w.block_tables)
    shared = po.paged_prefill_chunk(w.q, kc, vc, w.block_tables, [P] * S, [C] * S, bs, w.scale)
    # private pool: every sequence gets its own copy of the prefix
    per = P // bs + -(-C // bs)
    kc2, vc2 = torch.zeros(S * per * bs, 2, 16), torch.zeros(S * per * bs, 2, 16)
    tables2 = [np.arange(s * per, (s + 1) * per) for s in range(S)]
    for s in range(S):
        kc2[s * per * bs : s * per * bs + P] = w.k_prefix
        vc2[s * per * bs : s * per * bs + P] = w.v_prefix
        kc2[s * per * bs + P : s * per * bs + P + C] = w.k_chunk[s]
        vc2[s * per * bs + P : s * per * bs + P + C] = w.v_chunk[s]
    private = po.paged_prefill_chunk(w.q, kc2, vc2, tables2, [P] * S, [C] * S, bs, w.scale)
    np.testing.assert_allclose(shared, private, rtol=1e-12)


# ---------------------------------------------------------------- fp8
def test_e4m3_known_values():
    x = torch.tensor([464.0, 448.0, 2.0**-10, 2.0**-9, 1.0, -0.75, 0.0])
    y = x.to(torch.float8_e4m3fn).to(torch.float32)
    assert y.tolist() == [448.0, 448.0, 0.0, 2.0**-9, 1.0, -0.75, 0.0]
    assert torch.isnan(torch.tensor([480.0]).to(torch.float8_e4m3fn).to(torch.float32)).all()


def test_quantize_scales_and_roundtrip():
    rng = np.random.default_rng(13)
    bs, hkv, d, nb = 16, 2, 32, 3
    pool = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32))
    pool[bs : 2 * bs, 1] = 0.0  # an all-zero tile
    bits, scale = po.quantize_kv_e4m3(pool, bs)
    assert bits.dtype == torch.uint8 and scale.shape == (nb, hkv)
    amax = pool.reshape(nb, bs, hkv, d).abs().amax(dim=(1, 3))
    assert scale[1, 1] == 1.0
    mask = amax > 0
    assert torch.equal(scale[mask], (amax / 448.0)[mask])
    back = po.dequantize_kv_e4m3(bits, scale, bs)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 for normal values, absolute floor from the subnormals
    err = (back - pool).abs()
    bound = pool.abs() * 2.0**-4 + scale.repeat_interleave(bs, 0)[:, :, None] * 2.0**-10
    assert (err <= bound + 1e-12).all()
    # the tile maximum itself is stored exactly as +-448
    q = bits.view(torch.float8_e4m3fn).to(torch.float32).reshape(nb, bs, hkv, d).abs().amax(dim=(1, 3))
    assert (q[mask] == 448.0).all()


def test_fp8_decode_oracle_is_dequantise_then_attend():
    w = make_decode("c5", batch=2, len_range=(40, 90))
    kb, ks = po.quantize_kv_e4m3(w.k_pool, w.block_size)
    vb, vs = po.quantize_kv_e4m3(w.v_pool, w.block_size)
    kd, vd = po.dequantize_kv_e4m3(kb, ks, w.block_size), po.dequantize_kv_e4m3(vb, vs, w.block_size)
    tables = [t.tolist() for t in w.block_tables]
    approx = po.paged_decode(w.q, kd, vd, tables, w.seq_lens, w.block_size, w.scale)
    exact = po.paged_decode(w.q, w.k_pool, w.v_pool, tables, w.seq_lens, w.block_size, w.scale)
    assert np.abs(approx - exact).max() < 6e-2  # the quantisation error itself sits inside the fp8 tolerance
    assert np.abs(approx - exact).max() > 1e-4


# ---------------------------------------------------------------- fp8 append policy
def _empty_fp8_pool(nb, bs, hkv, d):
    return torch.zeros(nb * bs, hkv, d, dtype=torch.uint8), torch.ones(nb, hkv, dtype=torch.float32)


def test_fp8_append_of_whole_blocks_equals_block_quantisation():
    g = torch.Generator().manual_seed(11)
    nb, bs, hkv, d = 5, 16, 3, 32
    src = torch.randn(nb * bs, hkv, d, generator=g) * torch.logspace(-2, 1, nb * bs)[:, None, None]
    bits, scale = _empty_fp8_pool(nb, bs, hkv, d)
    perm = torch.randperm(nb * bs, generator=g).numpy()  # token t goes to slot perm[t]: every block completely
    po.append_kv_e4m3(bits, scale, src, perm, bs)
    pool = torch.empty_like(src)
    pool[perm] = src
    want_bits, want_scale = po.quantize_kv_e4m3(pool, bs)
    assert torch.equal(bits, want_bits) and torch.equal(scale, want_scale)


def test_fp8_append_token_by_token_policy():
    g = torch.Generator().manual_seed(12)
    bs, hkv, d = 16, 2, 64
    bits, scale = _empty_fp8_pool(2, bs, hkv, d)
    # block 0: magnitudes shrink -> the first row fixes the scale, earlier bytes never change
    rows = torch.randn(bs, hkv, d, generator=g) * torch.linspace(4.0, 0.5, bs)[:, None, None]
    rows = rows.clamp(-19.0, 19.0)
    rows[0, :, 0] = 20.0  # the tile maximum sits in the first row
    history = []
    for t in range(bs):
        po.append_kv_e4m3(bits, scale, rows[t : t + 1], [t], bs)
        history.append((bits[: t + 1].clone(), scale[0].clone()))
    for t in range(1, bs):
        assert torch.equal(history[t][0][:t], history[t - 1][0]) and torch.equal(history[t][1], history[0][1])
    assert torch.equal(scale[0], torch.full((hkv,), 20.0) / 448.0)
    # block 1: magnitudes grow -> the scale follows the running maximum and earlier rows are re-rounded
    rows = torch.randn(bs, hkv, d, generator=g) * torch.linspace(0.5, 4.0, bs)[:, None, None]
    for t in range(bs):
        po.append_kv_e4m3(bits, scale, rows[t : t + 1], [bs + t], bs)
        amax = rows[: t + 1].abs().amax(dim=(0, 2))
        assert torch.equal(scale[1], amax / 448.0)
    back = po.dequantize_kv_e4m3(bits, scale, bs)[bs:]
    # a row is rounded once when it is written and once more each time the tile maximum grows afterwards; every
    # rounding is within half an e4m3 step (2^-4 relative, 2^-10 of the scale grid for subnormals)
    run_max = torch.stack([rows[: t + 1].abs().amax(dim=(0, 2)) for t in range(bs)])  # [bs, hkv]
    grew = torch.cat([torch.zeros(1, hkv, dtype=torch.bool), run_max[1:] > run_max[:-1]])
    n_round = 1 + torch.stack([grew[t + 1 :].sum(0) for t in range(bs)])  # [bs, hkv]
    err = (back - rows).abs()
    bound = n_round[:, :, None] * (2.0 ** -4 * 1.01 * rows.abs() + scale[1][None, :, None] * 2.0 ** -9)
    assert (err <= bound).all(), float((err - bound).max())
    assert (n_round[0] > 3).all()  # the case does exercise repeated re-rounding


def test_fp8_append_restarts_a_recycled_block_and_skips_bad_slots():
    bs, hkv, d = 4, 1, 8
    bits, scale = _empty_fp8_pool(2, bs, hkv, d)
    po.append_kv_e4m3(bits, scale, torch.full((3, hkv, d), 100.0), [0, 1, 2], bs)
    assert float(scale[0, 0]) == float(np.float32(100.0) / np.float32(448.0))
    # the block is handed to another sequence: offset 0 is written again, the old rows do not count
    po.append_kv_e4m3(bits, scale, torch.full((2, hkv, d), 2.0), [0, -1], bs)
    assert float(scale[0, 0]) == float(np.float32(2.0) / np.float32(448.0))
    assert (bits[0].view(torch.float8_e4m3fn).to(torch.float32) == 448.0).all()
    po.append_kv_e4m3(bits, scale, torch.full((1, hkv, d), 1.0), [99], bs)  # outside the pool: ignored
    assert float(scale[1, 0]) == 1.0 and int(bits[bs:].max()) == 0


# ---------------------------------------------------------------- sliding window
def _swa_sdpa(q, k, v, scale, window):
    """The recipe of the reference's debug_swa.py (:56-82): tril mask AND (row - col) < window, SDPA with the
    explicit -inf mask.  q [B,T,Hq,D], k/v [B,T,Hkv,D] float32."""
    t = q.shape[1]
    n_rep = q.shape[2] // k.shape[2]
    row = torch.arange(t)[:, None]
    col = torch.arange(t)[None, :]
    keep = torch.tril(torch.ones(t, t, dtype=torch.bool)) & ((row - col) < window)
    mask = torch.where(keep, 0.0, float("-inf"))[None, None]
    qt = q.transpose(1, 2)
    kt = k.transpose(1, 2).repeat_interleave(n_rep, dim=1)
    vt = v.transpose(1, 2).repeat_interleave(n_rep, dim=1)
    return torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=mask, scale=scale).transpose(1, 2)


def test_window_prefill_matches_the_reference_recipe():
    g = torch.Generator().manual_seed(41)
    b, t, hq, hkv, d = 2, 16, 4, 2, 8  # debug_swa.py uses seq_len 16, window 4
    q, k, v = (torch.randn(b, t, h, d, generator=g) for h in (hq, hkv, hkv))
    scale = d ** -0.5
    for window in (1, 4, 7):
        want = _swa_sdpa(q, k, v, scale, window)
        np.testing.assert_allclose(po.dense_prefill(q, k, v, scale, window=window), want.numpy(), rtol=1e-4, atol=1e-4)
    # a window that covers the sequence is plain causal attention (debug_swa.py:131-150)
    np.testing.assert_allclose(po.dense_prefill(q, k, v, scale, window=t + 1), po.dense_prefill(q, k, v, scale),
                               rtol=0, atol=1e-12)
    assert not np.allclose(po.dense_prefill(q, k, v, scale, window=4), po.dense_prefill(q, k, v, scale))


def test_window_decode_is_the_last_row_of_windowed_prefill():
    g = torch.Generator().manual_seed(42)
    hq, hkv, d, bs, nb = 4, 2, 8, 4, 12
    lens = [13, 5, 1, 9]
    perm = torch.randperm(nb, generator=g).tolist()
    tables = [perm[0:4], perm[4:6], perm[6:7], perm[7:10]]
    kc = torch.randn(nb * bs, hkv, d, generator=g)
    vc = torch.randn(nb * bs, hkv, d, generator=g)
    q = torch.randn(len(lens), hq, d, generator=g)
    scale = 0.3
    for window in (1, 3, 6, 100):
        got = po.paged_decode(q, kc, vc, tables, lens, bs, scale, window=window)
        for b, n in enumerate(lens):
            slots = [tables[b][p // bs] * bs + p % bs for p in range(n)]
            qf = torch.zeros(1, n, hq, d)
            qf[0, -1] = q[b]
            want = _swa_sdpa(qf, kc[slots][None], vc[slots][None], scale, window)[0, -1]
            np.testing.assert_allclose(got[b], want.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(po.paged_decode(q, kc, vc, tables, lens, bs, scale, window=100),
                               po.paged_decode(q, kc, vc, tables, lens, bs, scale), rtol=0, atol=1e-12)
    # chunked prefill: rows [P:P+C] of the windowed dense result
    p_len, c_len, window = 7, 6, 5
    slots = [tables[0][p // bs] * bs + p % bs for p in range(p_len + c_len)]
    qc = torch.randn(1, c_len, hq, d, generator=g)
    qf = torch.cat([torch.zeros(1, p_len, hq, d), qc], 1)
    want = _swa_sdpa(qf, kc[slots][None], vc[slots][None], scale, window)[:, p_len:]
    got = po.paged_prefill_chunk(qc, kc, vc, [tables[0]], [p_len], [c_len], bs, scale, window=window)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-4, atol=1e-5)


def _reference_document_entry(boundaries, q_idx, kv_idx):
    """The loop of document_mask (attention/mask.py:173-186), one entry at a time."""
    q_doc = 0
    kv_doc = 0
    for i, boundary in enumerate(boundaries[1:]):
        if q_idx >= boundary:
            q_doc = i + 1
        if kv_idx >= boundary:
            kv_doc = i + 1
    return (q_doc == kv_doc) and (q_idx >= kv_idx)


def test_document_prefill_matches_the_explicit_mask_and_separate_documents():
    g = torch.Generator().manual_seed(43)
    b, t, hq, hkv, d = 2, 23, 4, 2, 8
    doc_lens = (5, 1, 0, 9, 4)  # sums to 19: positions 19..22 form one more document
    bounds = po.document_boundaries(doc_lens)
    assert bounds == [0, 5, 6, 6, 15, 19]
    assert po.document_of(bounds, np.arange(t)).tolist() == [0] * 5 + [1] + [3] * 9 + [4] * 4 + [5] * 4
    q, k, v = (torch.randn(b, t, h, d, generator=g) for h in (hq, hkv, hkv))
    scale = d ** -0.5
    keep = torch.tensor([[_reference_document_entry(bounds, r, c) for c in range(t)] for r in range(t)])
    mask = torch.where(keep, 0.0, float("-inf"))[None, None]
    n_rep = hq // hkv
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2).repeat_interleave(n_rep, dim=1),
        v.transpose(1, 2).repeat_interleave(n_rep, dim=1), attn_mask=mask, scale=scale).transpose(1, 2)
    got = po.dense_prefill(q, k, v, scale, doc_lens=doc_lens)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-4, atol=1e-5)
    # every document alone, plain causal
    for lo, hi in zip(bounds + [t], (bounds + [t])[1:]):
        if hi > lo:
            alone = po.dense_prefill(q[:, lo:hi], k[:, lo:hi], v[:, lo:hi], scale)
            np.testing.assert_allclose(got[:, lo:hi], alone, rtol=0, atol=1e-12)
    assert not np.allclose(got, po.dense_prefill(q, k, v, scale))
    # with a window on top: both bounds apply
    keep_w = keep & ((torch.arange(t)[:, None] - torch.arange(t)[None, :]) < 3)
    want_w = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2).repeat_interleave(n_rep, dim=1),
        v.transpose(1, 2).repeat_interleave(n_rep, dim=1),
        attn_mask=torch.where(keep_w, 0.0, float("-inf"))[None, None], scale=scale).transpose(1, 2)
    np.testing.assert_allclose(po.dense_prefill(q, k, v, scale, window=3, doc_lens=doc_lens), want_w.numpy(),
                               rtol=1e-4, atol=1e-5)
    # chunked: rows [P:P+C] of the packed result, documents by absolute position
    bs, p_len, c_len = 4, 9, 11
    nb = 6
    perm = torch.randperm(nb, generator=g).tolist()
    kc = torch.zeros(nb * bs, hkv, d)
    vc = torch.zeros(nb * bs, hkv, d)
    slots = [perm[p // bs] * bs + p % bs for p in range(p_len + c_len)]
    kc[slots] = k[0, : p_len + c_len]
    vc[slots] = v[0, : p_len + c_len]
    got_c = po.paged_prefill_chunk(q[:1, p_len : p_len + c_len], kc, vc, [perm], [p_len], [c_len], bs, scale,
                                   doc_lens=doc_lens)
    np.testing.assert_allclose(got_c, got[:1, p_len : p_len + c_len], rtol=0, atol=1e-12)


def test_rope_tables_closed_form():
    d, theta = 16, 10000.0
    pos = torch.tensor([[0, 1, 2, 77], [5, 4096, 3, 9]])
    cos, sin = po.rope_tables(pos, d, theta, torch.float32)
    assert cos.shape == (2, 4, d)
    angle = pos.numpy()[..., None].astype(np.float64) * theta ** (-np.arange(0, d, 2, dtype=np.float64) / d)
    np.testing.assert_allclose(cos[..., : d // 2].numpy(), np.cos(angle), atol=5e-4)  # float32 angles at 4096 rad
    np.testing.assert_allclose(sin[..., : d // 2].numpy(), np.sin(angle), atol=5e-4)
    small = pos.numpy() < 100
    np.testing.assert_allclose(cos[..., : d // 2].numpy()[small], np.cos(angle)[small], atol=1e-5)
    assert torch.equal(cos[..., : d // 2], cos[..., d // 2 :]) and torch.equal(sin[..., : d // 2], sin[..., d // 2 :])
    np.testing.assert_allclose((cos ** 2 + sin ** 2).numpy(), 1.0, atol=1e-6)
    assert torch.equal(cos[0, 0], torch.ones(d)) and torch.equal(sin[0, 0], torch.zeros(d))
    cb, _ = po.rope_tables(pos, d, theta, torch.bfloat16)
    assert cb.dtype == torch.bfloat16 and torch.equal(cb, cos.to(torch.bfloat16))  # cast once, at the end


def test_rope_literal_is_a_rotation():
    g = torch.Generator().manual_seed(44)
    n, h, d, theta = 9, 3, 16, 10000.0
    x = torch.randn(n, h, d, generator=g)
    pos = torch.tensor([[0, 1, 2, 3, 10, 50, 7, 7, 123]])
    cos, sin = (t[0] for t in po.rope_tables(pos, d, theta, torch.float32))
    angle = pos[0].numpy()[:, None].astype(np.float64) * theta ** (-np.arange(0, d, 2, dtype=np.float64) / d)
    got = po.rope_literal(x, cos, sin)
    np.testing.assert_allclose(got.numpy(), po.rope_exact(x, angle), atol=2e-5)
    assert torch.equal(got[0], x[0])  # position 0
    pair_norm = lambda t: (t[..., : d // 2] ** 2 + t[..., d // 2 :] ** 2)
    np.testing.assert_allclose(pair_norm(got).numpy(), pair_norm(x).numpy(), rtol=1e-5, atol=1e-6)
    # a sign or half mix-up fails this: rotating by +angle then by -angle is the identity
    back = po.rope_literal(got, cos, -sin)
    np.testing.assert_allclose(back.numpy(), x.numpy(), atol=1e-5)
    # relative positions: <rope(q, m), rope(k, n)> depends on m - n only
    q, k = torch.randn(1, 1, d, generator=g), torch.randn(1, 1, d, generator=g)
    def dot(m, nn):
        c, s = (t[0] for t in po.rope_tables(torch.tensor([[m, nn]]), d, theta, torch.float32))
        return float((po.rope_literal(q, c[:1], s[:1]) * po.rope_literal(k, c[1:], s[1:])).sum())
    assert abs(dot(5, 2) - dot(40, 37)) < 1e-4 and abs(dot(5, 2) - dot(2, 5)) > 1e-3
    # bf16: every product and the sum rounded to bf16 -> within a few bf16 ulps of the exact rotation
    xb = x.to(torch.bfloat16)
    gb = po.rope_literal(xb, cos.to(torch.bfloat16), sin.to(torch.bfloat16))
    assert gb.dtype == torch.bfloat16
    np.testing.assert_allclose(gb.float().numpy(), po.rope_exact(xb, angle), atol=0.06, rtol=0.02)


# ---------------------------------------------------------------- arbitrary masks
def test_masked_attention_against_sdpa_with_a_boolean_mask_and_the_causal_case():
    """paged_attend_masked: (1) the library routine with attn_mask on the gathered, head-expanded tensors
    (rows with at least one kept key); (2) a row that keeps nothing gives zeros; (3) keys past the context end
    are zero rows that still take softmax mass when kept (the reference's padded decode gather); (4) with the
    causal predicate it is the chunked prefill of the other checker function; (5) a head-dependent mask uses each
    head's own row."""
    rng = np.random.default_rng(41)
    bs, hq, hkv, d = 4, 4, 2, 8
    kc, vc = _tiny_pool(rng, num_blocks=8, bs=bs, hkv=hkv, d=d)
    tables = [[5, 2, 7], [1, 3]]
    ctx, ql = [10, 7], [3, 2]
    n_keys = 12
    q = torch.from_numpy(rng.standard_normal((2, 3, hq, d)).astype(np.float32))
    keep = rng.random((2, 3, hq, n_keys)) < 0.5
    keep[0, 1] = False          # a row that keeps nothing
    keep[1, 0, :, 7:] = True    # keys past the context end (7) kept
    got = po.paged_attend_masked(q, kc, vc, tables, ctx, ql, keep, bs, 0.3)
    kg, vg = po.kv_gather_padded(kc, vc, [t + [0] * 3 for t in tables], [n_keys, n_keys], bs)
    for b in range(2):
        kb, vb = kg[b].clone(), vg[b].clone()
        kb[ctx[b]:] = 0
        vb[ctx[b]:] = 0
        for t in range(ql[b]):
            for h in range(hq):
                if not keep[b, t, h].any():
                    assert not got[b, t, h].any()
                    continue
                want = F.scaled_dot_product_attention(
                    q[b, t, h][None, None].double(), kb[:, h // 2][None].double(), vb[:, h // 2][None].double(),
                    attn_mask=torch.from_numpy(keep[b, t, h])[None, None], scale=0.3)
                np.testing.assert_allclose(got[b, t, h], want[0, 0].numpy(), rtol=1e-9, atol=1e-12)
    assert not got[1, 2].any()  # past q_lens
    # (3) zero keys take mass: dropping them from the mask changes the row
    keep2 = keep.copy()
    keep2[1, 0, :, 7:] = False
    assert np.abs(po.paged_attend_masked(q, kc, vc, tables, ctx, ql, keep2, bs, 0.3)[1, 0] - got[1, 0]).max() > 1e-3
    # (4) the causal predicate over a prefix: chunk row t sits at position P + t
    prefix = [c - n for c, n in zip(ctx, ql)]
    causal = np.zeros((2, 3, 1, n_keys), dtype=bool)
    for b in range(2):
        for t in range(ql[b]):
            causal[b, t, 0, : prefix[b] + t + 1] = True
    np.testing.assert_allclose(po.paged_attend_masked(q, kc, vc, tables, ctx, ql, causal, bs, 0.3),
                               po.paged_prefill_chunk(q, kc, vc, tables, prefix, ql, bs, 0.3), rtol=1e-10, atol=1e-12)
