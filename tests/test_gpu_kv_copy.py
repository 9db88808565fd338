"""KV append (scatter) and block-table gather on the GPU: bit-exact against the CPU checker."""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import ops
from research_amd.workloads import make_decode, make_prefill_c3
from tests.gpu_helpers import DEV, announce, tables_to_device

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.cpu().view(torch.uint8) if t.dtype != torch.uint8 else t.cpu()


def _scatter_case(dtype, hkv, d, n_slots, slots, seed):
    rng = np.random.default_rng(seed)
    n = len(slots)
    k = torch.from_numpy(rng.standard_normal((n, hkv, d)).astype(np.float32)).to(dtype)
    v = torch.from_numpy(rng.standard_normal((n, hkv, d)).astype(np.float32)).to(dtype)
    kc0 = torch.from_numpy(rng.standard_normal((n_slots, hkv, d)).astype(np.float32)).to(dtype)
    vc0 = torch.from_numpy(rng.standard_normal((n_slots, hkv, d)).astype(np.float32)).to(dtype)
    ek, ev = kc0.clone(), vc0.clone()
    keep = [s if 0 <= s < n_slots else -1 for s in slots]
    po.kv_scatter(ek, ev, k, v, keep)
    kc, vc = kc0.to(DEV), vc0.to(DEV)
    ops.kv_scatter(kc, vc, k.to(DEV), v.to(DEV), torch.tensor(slots, dtype=torch.int64, device=DEV))
    torch.cuda.synchronize()
    assert torch.equal(_bits(kc), _bits(ek)) and torch.equal(_bits(vc), _bits(ev))


def test_scatter_reference_round_trip():
    """Slots 0..3 receive rows 0..3 (the reference's own store check, test_kv_cache.py:101-111)."""
    announce("scatter reference round trip")
    torch.manual_seed(0)
    k = torch.randn(4, 4, 32, dtype=torch.bfloat16)
    v = torch.randn(4, 4, 32, dtype=torch.bfloat16)
    kc = torch.zeros(64, 4, 32, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    ops.kv_scatter(kc, vc, k.to(DEV), v.to(DEV), torch.arange(4, device=DEV))
    assert torch.equal(kc[0].cpu(), k[0]) and torch.equal(vc[3].cpu(), v[3]) and not kc[4:].any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16, torch.uint8])
def test_scatter_drops_negative_and_out_of_range_slots(dtype):
    announce(f"scatter skip slots {dtype}")
    slots = [5, -1, 0, 17, -7, 9, 2, 23, 24, 1 << 40]
    if dtype == torch.uint8:
        rng = np.random.default_rng(3)
        k = torch.from_numpy(rng.integers(0, 256, (len(slots), 2, 16), dtype=np.uint8))
        kc0 = torch.from_numpy(rng.integers(0, 256, (24, 2, 16), dtype=np.uint8))
        ek, ev = kc0.clone(), kc0.clone()
        po.kv_scatter(ek, ev, k, k, [s if 0 <= s < 24 else -1 for s in slots])
        kc, vc = kc0.to(DEV), kc0.to(DEV)
        ops.kv_scatter(kc, vc, k.to(DEV), k.to(DEV), torch.tensor(slots, dtype=torch.int64, device=DEV))
        assert torch.equal(kc.cpu(), ek) and torch.equal(vc.cpu(), ev)
    else:
        _scatter_case(dtype, 2, 8, 24, slots, seed=4)


def test_scatter_rows_not_multiple_of_16_bytes():
    announce("scatter 4-byte path")
    _scatter_case(torch.bfloat16, 1, 6, 40, [3, 39, -1, 0, 12], seed=5)  # 12-byte rows


def test_scatter_c3_append_full_size():
    """workload c3 append: 32 x 256 new tokens into a 640-block pool next to a shared prefix."""
    announce("scatter c3 full size")
    w = make_prefill_c3()
    shape = (w.num_blocks * w.block_size, w.num_kv_heads, w.head_dim)
    ek, ev = torch.zeros(shape, dtype=w.dtype), torch.zeros(shape, dtype=w.dtype)
    ek[torch.from_numpy(w.prefix_slots())] = w.k_prefix
    ev[torch.from_numpy(w.prefix_slots())] = w.v_prefix
    kc, vc = ek.to(DEV), ev.to(DEV)
    slots = w.chunk_slots()
    assert len(set(slots.tolist())) == len(slots) == 8192
    ek[torch.from_numpy(slots)] = w.k_chunk.reshape(-1, *shape[1:])  # closed form of the append
    ev[torch.from_numpy(slots)] = w.v_chunk.reshape(-1, *shape[1:])
    ops.kv_scatter(kc, vc, w.k_chunk.reshape(-1, *shape[1:]).to(DEV), w.v_chunk.reshape(-1, *shape[1:]).to(DEV),
                   torch.from_numpy(slots).to(DEV))
    assert torch.equal(_bits(kc), _bits(ek)) and torch.equal(_bits(vc), _bits(ev))
    # round trip through the gather: every sequence reads back prefix + its own chunk
    lens = [w.prefix_len + w.chunk_len] * w.num_seqs
    kg, vg = ops.kv_gather(kc, vc, tables_to_device(w.block_tables),
                           torch.tensor(lens, dtype=torch.int32, device=DEV), lens[0], w.block_size)
    for s in (0, 7, 31):
        assert torch.equal(_bits(kg[s, : w.prefix_len]), _bits(w.k_prefix))
        assert torch.equal(_bits(vg[s, w.prefix_len :]), _bits(w.v_chunk[s]))


@pytest.mark.parametrize("name,kw", [("c1", {}), ("c2", dict(batch=6, len_range=(100, 700)))])
def test_gather_matches_oracle(name, kw):
    announce(f"gather {name} {kw}")
    w = make_decode(name, **kw)
    tables = [t.tolist() for t in w.block_tables]
    ek, ev = po.kv_gather_padded(w.k_pool, w.v_pool, tables, w.seq_lens, w.block_size)
    kg, vg = ops.kv_gather(w.k_pool.to(DEV), w.v_pool.to(DEV), tables_to_device(tables),
                           torch.from_numpy(w.seq_lens.astype(np.int32)).to(DEV), int(w.seq_lens.max()), w.block_size)
    assert torch.equal(_bits(kg), _bits(ek)) and torch.equal(_bits(vg), _bits(ev))


def test_gather_short_table_and_bad_ids_read_as_zero():
    announce("gather short table / bad ids")
    rng = np.random.default_rng(6)
    bs, hkv, d, nb = 4, 2, 8, 6
    kc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32))
    vc = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32))
    tables, lens = [(3, 0, 5), (2,), (4, 1)], [10, 7, 0]
    ek, ev = po.kv_gather_padded(kc, vc, tables, lens, bs)
    kg, vg = ops.kv_gather(kc.to(DEV), vc.to(DEV), tables_to_device(tables),
                           torch.tensor(lens, dtype=torch.int32, device=DEV), 10, bs)
    assert torch.equal(kg.cpu(), ek) and torch.equal(vg.cpu(), ev)
    # block ids outside the pool read as zeros instead of faulting
    bad = torch.tensor([[3, 99, -5]], dtype=torch.int32, device=DEV)
    kg, _ = ops.kv_gather(kc.to(DEV), vc.to(DEV), bad, torch.tensor([12], dtype=torch.int32, device=DEV), 12, bs)
    assert torch.equal(kg[0, :4].cpu(), kc[12:16]) and not kg[0, 4:].any()


# ---------------------------------------------------------------- fp8 append
def _fp8_pool(nb, bs, hkv, d):
    bits = torch.zeros(nb * bs, hkv, d, dtype=torch.uint8)
    scale = torch.ones(nb, hkv, dtype=torch.float32)
    return bits, scale


def _append_both(bits, scale, src, slots, bs):
    """The same append on the device (through the C ABI) and in the checker; returns the device result."""
    kb = bits.clone().to(DEV).view(torch.float8_e4m3fn)
    vb = bits.clone().to(DEV).view(torch.float8_e4m3fn)
    ks, vs = scale.clone().to(DEV), scale.clone().to(DEV)
    sl = torch.from_numpy(np.asarray(slots, dtype=np.int64)).to(DEV)
    ops.kv_append_e4m3(kb, vb, ks, vs, src.to(DEV), (src * 0.5).to(DEV), sl, bs)
    po.append_kv_e4m3(bits, scale, src, slots, bs)
    assert torch.equal(kb.view(torch.uint8).cpu(), bits), "K bytes differ from the checker"
    assert torch.equal(ks.cpu(), scale), "K scales differ from the checker"
    return kb, vb, ks, vs


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_fp8_append_bit_exact_token_by_token_and_in_chunks(dtype):
    announce(f"fp8 append {dtype}")
    g = torch.Generator().manual_seed(21)
    nb, bs, hkv, d = 6, 16, 8, 128
    bits, scale = _fp8_pool(nb, bs, hkv, d)
    # a prompt of 37 tokens into blocks 4, 1, 5 in one call, then 20 decode steps one token at a time with
    # growing magnitude (every step re-rounds the last block), then a chunk that crosses into a new block
    table = [4, 1, 5, 0, 2]
    pos_slot = lambda p: table[p // bs] * bs + p % bs
    prompt = (torch.randn(37, hkv, d, generator=g) * 0.3).to(dtype)
    _append_both(bits, scale, prompt, [pos_slot(p) for p in range(37)], bs)
    for i in range(20):
        row = (torch.randn(1, hkv, d, generator=g) * (0.3 + 0.2 * i)).to(dtype)
        _append_both(bits, scale, row, [pos_slot(37 + i)], bs)
    chunk = (torch.randn(11, hkv, d, generator=g) * 3).to(dtype)
    _append_both(bits, scale, chunk, [pos_slot(57 + i) for i in range(11)], bs)
    # the V pool of the same calls holds half the values: same bytes, half the scale (powers of two are exact)
    # and the dequantised pool is close to what was appended
    everything = prompt.float()
    back = po.dequantize_kv_e4m3(bits, scale, bs)
    got = torch.stack([back[pos_slot(p)] for p in range(37)])
    assert ((got - everything).abs() <= 0.5 * everything.abs() + 0.05).all()


def test_fp8_append_v_pool_and_edge_cases():
    announce("fp8 append edge cases")
    g = torch.Generator().manual_seed(22)
    nb, bs, hkv, d = 4, 16, 2, 64
    bits, scale = _fp8_pool(nb, bs, hkv, d)
    src = torch.randn(5, hkv, d, generator=g).to(torch.bfloat16)
    # negative and out-of-pool slots are skipped, a duplicated slot keeps the later token
    kb, vb, ks, vs = _append_both(bits, scale, src, [3 * bs, -1, nb * bs + 7, 3 * bs + 1, 3 * bs + 1], bs)
    # the V rows of these calls are half the K rows: same bytes, half the scale (exact), other tiles untouched
    assert torch.equal(vb.view(torch.uint8).cpu(), bits)
    assert torch.equal(vs.cpu()[3], scale[3] * 0.5) and (vs.cpu()[:3] == 1).all() and (scale[:3] == 1).all()
    # whole blocks at once equal the block quantiser
    full = torch.randn(2 * bs, hkv, d, generator=g)
    bits2, scale2 = _fp8_pool(nb, bs, hkv, d)
    _append_both(bits2, scale2, full, list(range(bs, 3 * bs)), bs)
    want_bits, want_scale = po.quantize_kv_e4m3(full, bs)
    assert torch.equal(bits2[bs : 3 * bs], want_bits) and torch.equal(scale2[1:3], want_scale)
    # nothing to do
    ops.kv_append_e4m3(kb, vb, ks, vs, src[:0].to(DEV), src[:0].to(DEV), torch.zeros(0, dtype=torch.int64, device=DEV), bs)


@pytest.mark.parametrize("hkv,d,bs,dtype", [
    (12, 64, 16, torch.bfloat16),   # more kv heads than a workgroup's eight groups of lanes: two passes
    (3, 256, 32, torch.float16),    # tiles larger than a lane keeps in registers
    (1, 128, 16, torch.float32),    # one kv head: a single group of lanes works
    (5, 20, 8, torch.bfloat16),     # head_dim not a multiple of 8: the element-wise kernel
])
def test_fp8_append_shapes(hkv, d, bs, dtype):
    """The append kernels over head counts, head dims and block sizes: bytes and scales against the checker's
    statement of the policy, for a prompt written in one call and growth over the following calls."""
    announce(f"fp8 append shapes hkv={hkv} d={d} bs={bs} {dtype}")
    g = torch.Generator().manual_seed(23 + hkv)
    nb = 7
    bits, scale = _fp8_pool(nb, bs, hkv, d)
    kc = bits.clone().view(torch.float8_e4m3fn).to(DEV)
    vc = bits.clone().view(torch.float8_e4m3fn).to(DEV)
    ks, vs = scale.clone().to(DEV), scale.clone().to(DEV)
    vbits, vscale = bits.clone(), scale.clone()
    table = [4, 1, 6, 0, 3]
    at = 0
    for n_new, gain in ((2 * bs + 3, 1.0), (1, 4.0), (bs - 5, 0.5), (bs + 2, 9.0)):
        pos = list(range(at, at + n_new))
        at += n_new
        slots = torch.tensor([table[p // bs] * bs + p % bs for p in pos])
        k = (torch.randn(n_new, hkv, d, generator=g) * gain).to(dtype)
        v = (torch.randn(n_new, hkv, d, generator=g) * gain).to(dtype)
        po.append_kv_e4m3(bits, scale, k, slots.tolist(), bs)
        po.append_kv_e4m3(vbits, vscale, v, slots.tolist(), bs)
        ops.kv_append_e4m3(kc, vc, ks, vs, k.to(DEV), v.to(DEV), slots.to(DEV), bs)
        assert torch.equal(kc.cpu().view(torch.uint8), bits) and torch.equal(ks.cpu(), scale)
        assert torch.equal(vc.cpu().view(torch.uint8), vbits) and torch.equal(vs.cpu(), vscale)


def test_fp8_append_with_and_without_the_row_index():
    """The append with the index of rows by touched block (what ops.touched_blocks builds), with a bare list of
    blocks (every workgroup scans the slot list) and with the list in another order than the index's sort: the
    same bytes and scales, on a shuffled slot list with skipped rows and a slot written twice."""
    announce("fp8 append row index")
    g = torch.Generator().manual_seed(31)
    nb, bs, hkv, d = 40, 16, 4, 128
    n = 500
    slots = torch.randperm(nb * bs, generator=g)[:n]
    slots[7] = -1
    slots[300] = nb * bs + 3
    slots[450] = slots[20]  # written twice: the later row is stored
    k = torch.randn(n, hkv, d, generator=g).to(torch.bfloat16)
    v = torch.randn(n, hkv, d, generator=g).to(torch.bfloat16)
    results = []
    for mode in ("index", "scan", "reordered"):
        bits, scale = _fp8_pool(nb, bs, hkv, d)
        kc = bits.clone().view(torch.float8_e4m3fn).to(DEV)
        vc = bits.clone().view(torch.float8_e4m3fn).to(DEV)
        ks, vs = scale.clone().to(DEV), scale.clone().to(DEV)
        touched = ops.touched_blocks(slots.to(DEV), bs, nb)
        assert int(touched.block_start[-1]) == n - 2 and touched.row_order.numel() == n - 2
        if mode == "scan":
            touched = touched.blocks
        elif mode == "reordered":
            perm = torch.randperm(touched.blocks.numel(), generator=g).to(DEV)
            counts = (touched.block_start[1:] - touched.block_start[:-1])[perm]
            start = torch.zeros_like(touched.block_start)
            start[1:] = torch.cumsum(counts, 0)
            order = torch.cat([touched.row_order[int(touched.block_start[i]): int(touched.block_start[i + 1])]
                               for i in perm.tolist()])
            touched = ops.TouchedBlocks(touched.blocks[perm].contiguous(), order.contiguous(), start)
        ops.kv_append_e4m3(kc, vc, ks, vs, k.to(DEV), v.to(DEV), slots.to(DEV), bs, touched)
        results.append((kc.cpu().view(torch.uint8), vc.cpu().view(torch.uint8), ks.cpu(), vs.cpu()))
    want_bits, want_scale = _fp8_pool(nb, bs, hkv, d)
    po.append_kv_e4m3(want_bits, want_scale, k, slots.tolist(), bs)
    for got in results:
        assert torch.equal(got[0], want_bits) and torch.equal(got[2], want_scale)
        for a, b in zip(got, results[0]):
            assert torch.equal(a, b)
