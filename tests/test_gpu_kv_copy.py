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
    """BASELINE config 3 append: 32 x 256 new tokens into a 640-block pool next to a shared prefix."""
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
