"""Paged decode attention on the GPU against the CPU checker, through the C ABI.

Tolerances (absolute on |want|<=1, relative above): 1e-5 for the fp32 pool,
2e-2 for bf16/fp16 pools with fp32 accumulation, 6e-2 for the fp8-e4m3 pool
against dequantise-then-attend.
"""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import ops
from research_amd.workloads import make_decode
from tests.gpu_helpers import DEV, announce, assert_close, run_decode, tables_to_device

pytestmark = pytest.mark.gpu


def _lists(w):
    return [t.tolist() for t in w.block_tables]


def _gpu_decode(w, **kw):
    return run_decode(w.q.to(DEV), w.k_pool.to(DEV), w.v_pool.to(DEV), _lists(w), w.seq_lens, w.block_size, w.scale,
                      **kw)


def test_c1_fp32_masked_and_pad_zero_keys():
    """workload c1 in both semantics; the padded one against the literal restatement too."""
    announce("decode c1 fp32")
    w = make_decode("c1")
    want = po.paged_decode(w.q, w.k_pool, w.v_pool, _lists(w), w.seq_lens, w.block_size, w.scale)
    assert_close(_gpu_decode(w), want, 1e-5, "c1 masked")
    pad = (w.seq_lens.max() - w.seq_lens).tolist()
    got = _gpu_decode(w, extra_zero=pad)
    want = po.paged_decode(w.q, w.k_pool, w.v_pool, _lists(w), w.seq_lens, w.block_size, w.scale, pad_zero_keys=True)
    assert_close(got, want, 1e-5, "c1 pad_zero_keys")
    lit = po.decode_literal(w.q[:, None], w.k_pool, w.v_pool, _lists(w), w.seq_lens, w.block_size, w.scale,
                            vectorised_gather=True)[:, 0]
    assert_close(got, lit, 1e-5, "c1 vs literal reference restatement")


def test_c2_bf16_full_size():
    """workload c2 at full size (B=64, 141 622 keys)."""
    announce("decode c2 bf16 full")
    w = make_decode("c2")
    assert w.total_tokens == 141622
    want = po.paged_decode(w.q, w.k_pool, w.v_pool, _lists(w), w.seq_lens, w.block_size, w.scale)
    assert_close(_gpu_decode(w), want, 2e-2, "c2")


def test_c4_shape_reduced_batch():
    """workload c4's shape (Hq=32, Hkv=8, D=128, lognormal lengths) on 24 sequences."""
    announce("decode c4 reduced")
    w = make_decode("c4", batch=24, len_range=(64, 6000))
    want = po.paged_decode(w.q, w.k_pool, w.v_pool, _lists(w), w.seq_lens, w.block_size, w.scale)
    assert_close(_gpu_decode(w), want, 2e-2, "c4 reduced")


def test_result_does_not_depend_on_the_partition():
    """Where the workgroup ranges cut the sequences depends on the batch around them:
    alone, every sequence is split over the whole grid; in the batch most are whole."""
    announce("decode partition invariance")
    w = make_decode("c4", batch=12, len_range=(64, 5000), seed=77)
    tables = _lists(w)
    q, kp, vp = w.q.to(DEV), w.k_pool.to(DEV), w.v_pool.to(DEV)
    together = run_decode(q, kp, vp, tables, w.seq_lens, w.block_size, w.scale).float()
    want = po.paged_decode(w.q, w.k_pool, w.v_pool, tables, w.seq_lens, w.block_size, w.scale)
    assert_close(together, want, 2e-2, "batch")
    for b in range(w.batch):
        alone = run_decode(q[b : b + 1], kp, vp, tables[b : b + 1], w.seq_lens[b : b + 1], w.block_size, w.scale)
        assert_close(alone.float(), together[b : b + 1], 1e-2, f"sequence {b} alone")
    order = list(range(w.batch))[::-1]
    rev = run_decode(q[order], kp, vp, [tables[i] for i in order], w.seq_lens[order], w.block_size, w.scale).float()
    assert_close(rev, together[order], 1e-2, "reversed batch")


def test_long_single_sequence_is_split_over_the_grid():
    """One 40 000-key sequence: thousands of blocks, every workgroup gets a piece, one merged row."""
    announce("decode single long sequence")
    w = make_decode("c2", batch=1, len_range=(40000, 40000), seed=9)
    want = po.paged_decode(w.q, w.k_pool, w.v_pool, _lists(w), w.seq_lens, w.block_size, w.scale)
    assert_close(_gpu_decode(w), want, 2e-2, "single long sequence")


def test_pool_permutation_and_constant_values():
    announce("decode permutation / constant V")
    w = make_decode("c2", batch=5, len_range=(30, 400), seed=5)
    base = _gpu_decode(w).float()
    rng = np.random.default_rng(0)
    perm = rng.permutation(w.num_blocks)  # new id of block i is perm[i]
    src = torch.from_numpy(np.argsort(perm))  # block living at new position j
    bs = w.block_size
    k2 = w.k_pool.reshape(w.num_blocks, bs, *w.k_pool.shape[1:])[src].reshape(w.k_pool.shape)
    v2 = w.v_pool.reshape(w.num_blocks, bs, *w.v_pool.shape[1:])[src].reshape(w.v_pool.shape)
    tables2 = [perm[t].tolist() for t in w.block_tables]
    moved = run_decode(w.q.to(DEV), k2.to(DEV), v2.to(DEV), tables2, w.seq_lens, bs, w.scale).float()
    assert torch.equal(moved, base)  # same arithmetic in the same order: bit-identical
    row = torch.linspace(-2, 2, w.head_dim).to(w.dtype)
    vconst = row.expand_as(w.v_pool).contiguous()
    out = run_decode(w.q.to(DEV), w.k_pool.to(DEV), vconst.to(DEV), _lists(w), w.seq_lens, bs, w.scale)
    assert_close(out, row.float().expand(w.batch, w.num_q_heads, w.head_dim), 1e-2, "constant V")


@pytest.mark.parametrize("hq,hkv,d,dtype", [
    (14, 2, 64, torch.bfloat16),   # group of 7 (Qwen2.5-0.5B), padded to 8 in the kernel
    (8, 4, 32, torch.bfloat16),    # the reference script's shape (test_kv_cache.py:131-136)
    (6, 6, 128, torch.float16),    # MHA, 6 kv heads: two per wave load
    (3, 1, 256, torch.bfloat16),   # MQA, group of 3, D=256
    (16, 8, 256, torch.bfloat16),  # Gemma-2-9B-like: D=256 rows span 32 lanes, two kv heads per wave load
    (8, 2, 256, torch.float16),    # D=256, group of 4
    (32, 2, 128, torch.float32),   # group of 16: two passes of 8
    (5, 5, 64, torch.float32),     # odd head count: one kv head per wave load
    (10, 2, 80, torch.bfloat16),   # head sizes between the compiled ones: the next larger kernel, idle lanes masked
    (6, 3, 96, torch.float16),
    (4, 1, 112, torch.bfloat16),
    (8, 2, 160, torch.bfloat16),
    (6, 2, 192, torch.float16),
    (4, 2, 40, torch.float32),
    (4, 2, 24, torch.bfloat16),
    (2, 2, 8, torch.float32),
])
def test_head_layouts(hq, hkv, d, dtype):
    announce(f"decode heads hq={hq} hkv={hkv} d={d} {dtype}")
    rng = np.random.default_rng(hq * 1000 + d)
    bs, nb = 4, 64
    lens = [37, 1, 100, 64, 5]
    perm = rng.permutation(nb)
    tables, at = [], 0
    for n in lens:
        c = -(-n // bs)
        tables.append(perm[at : at + c].tolist())
        at += c
    q = torch.from_numpy(rng.standard_normal((len(lens), hq, d)).astype(np.float32)).to(dtype)
    kp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
    vp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
    want = po.paged_decode(q, kp, vp, tables, lens, bs, d**-0.5)
    got = run_decode(q.to(DEV), kp.to(DEV), vp.to(DEV), tables, lens, bs, d**-0.5)
    assert_close(got, want, 1e-5 if dtype == torch.float32 else 2e-2, "head layout")


def test_edge_cases_empty_short_table_and_garbage_tail():
    announce("decode edge cases")
    rng = np.random.default_rng(21)
    bs, nb, hq, hkv, d = 16, 12, 8, 2, 64
    q = torch.from_numpy(rng.standard_normal((4, hq, d)).astype(np.float32))
    kp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32))
    vp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32))
    tables = [[3, 7], [], [5], [9, 1, 0]]
    lens = [20, 0, 40, 33]  # seq 1 empty; seq 2's table covers 16 of its 40 keys
    # poison everything past each sequence's length inside its last block: must never be read as a key
    kp[7 * bs + 4 : 8 * bs] = float("nan")
    vp[7 * bs + 4 : 8 * bs] = float("inf")
    kp[0 * bs + 1 : 1 * bs] = float("nan")
    vp[0 * bs + 1 : 1 * bs] = float("nan")
    want = po.paged_decode(q, kp, vp, tables, lens, bs, 0.125)
    got = run_decode(q.to(DEV), kp.to(DEV), vp.to(DEV), tables, lens, bs, 0.125)
    assert_close(got, want, 1e-5, "edge")
    assert not got[1].any()  # empty sequence -> zeros
    lit = po.decode_literal(q[2:3, None], kp, vp, tables[2:3], lens[2:3], bs, 0.125)[:, 0]
    assert_close(got[2:3], lit, 1e-5, "short table vs literal restatement")


def test_block_ids_outside_the_pool_do_not_fault():
    announce("decode bad block ids")
    rng = np.random.default_rng(22)
    bs, nb = 16, 4
    q = torch.from_numpy(rng.standard_normal((1, 4, 64)).astype(np.float32))
    kp = torch.from_numpy(rng.standard_normal((nb * bs, 2, 64)).astype(np.float32))
    vp = torch.from_numpy(rng.standard_normal((nb * bs, 2, 64)).astype(np.float32))
    got = run_decode(q.to(DEV), kp.to(DEV), vp.to(DEV), [[2, 1000, -3]], [48], bs, 0.125)
    want = po.paged_decode(q, kp, vp, [[2]], [48], bs, 0.125)  # the two bad blocks act as missing ones
    assert_close(got, want, 1e-5, "bad ids")


def test_quantize_matches_torch_e4m3_bit_for_bit():
    announce("quantize e4m3")
    w = make_decode("c5", batch=3, len_range=(50, 300))
    w.k_pool[5 * 16 : 6 * 16, 3] = 0  # an all-zero tile
    for src in (w.k_pool, w.v_pool.float(), w.v_pool.to(torch.float16)):
        bits, scale = ops.quantize_kv_e4m3(src.to(DEV), w.block_size)
        eb, es = po.quantize_kv_e4m3(src, w.block_size)
        assert torch.equal(scale.cpu(), es)
        assert torch.equal(bits.cpu().view(torch.uint8), eb)


def test_c5_fp8_reduced():
    """workload c5's shape with shorter contexts: e4m3 pool, per-(block, head) scales, bf16 q."""
    announce("decode c5 fp8 reduced")
    w = make_decode("c5", batch=4, len_range=(3000, 9000))
    kb, ks = ops.quantize_kv_e4m3(w.k_pool.to(DEV), w.block_size)
    vb, vs = ops.quantize_kv_e4m3(w.v_pool.to(DEV), w.block_size)
    kd = po.dequantize_kv_e4m3(kb.cpu().view(torch.uint8), ks.cpu(), w.block_size)
    vd = po.dequantize_kv_e4m3(vb.cpu().view(torch.uint8), vs.cpu(), w.block_size)
    want = po.paged_decode(w.q, kd, vd, _lists(w), w.seq_lens, w.block_size, w.scale)
    got = run_decode(w.q.to(DEV), kb, vb, _lists(w), w.seq_lens, w.block_size, w.scale, k_scale=ks, v_scale=vs)
    assert_close(got, want, 6e-2, "c5 fp8")
    assert_close(got, want, 2e-2, "c5 fp8 (the arithmetic itself is as tight as bf16)")


@pytest.mark.parametrize("window", [1, 16, 17, 100, 1000, 5000])
def test_sliding_window_decode(window):
    """Only the last `window` keys count; blocks wholly before the window are not visited."""
    announce(f"decode window {window}")
    w = make_decode("c4", batch=9, len_range=(1, 3000), seed=13)
    q, kp, vp = w.q.to(DEV), w.k_pool.to(DEV), w.v_pool.to(DEV)
    tables = tables_to_device(_lists(w))
    lens = torch.from_numpy(w.seq_lens.astype(np.int32)).to(DEV)
    ws = ops.decode_workspace(q, kp)
    got = ops.decode(q, kp, vp, tables, lens, w.block_size, w.scale, ws, window=window)
    want = po.paged_decode(w.q, w.k_pool, w.v_pool, _lists(w), w.seq_lens, w.block_size, w.scale, window=window)
    assert_close(got, want, 2e-2, f"window {window}")
    if window >= int(w.seq_lens.max()):
        assert torch.equal(got, ops.decode(q, kp, vp, tables, lens, w.block_size, w.scale, ws))


def test_sliding_window_decode_other_types_and_garbage_before_the_window():
    announce("decode window fp32 / fp8 / poisoned prefix")
    w = make_decode("c1")
    lists = _lists(w)
    got = run_decode(w.q.to(DEV), w.k_pool.to(DEV), w.v_pool.to(DEV), lists, w.seq_lens, w.block_size, w.scale)
    q, kp, vp = w.q.to(DEV), w.k_pool.to(DEV), w.v_pool.to(DEV)
    tables = tables_to_device(lists)
    lens = torch.from_numpy(w.seq_lens.astype(np.int32)).to(DEV)
    ws = ops.decode_workspace(q, kp)
    for window in (3, 20):
        got = ops.decode(q, kp, vp, tables, lens, w.block_size, w.scale, ws, window=window)
        want = po.paged_decode(w.q, w.k_pool, w.v_pool, lists, w.seq_lens, w.block_size, w.scale, window=window)
        assert_close(got, want, 1e-5, f"c1 window {window}")
    w = make_decode("c5", batch=3, len_range=(200, 900))
    k8, ks = ops.quantize_kv_e4m3(w.k_pool.to(DEV), w.block_size)
    v8, vs = ops.quantize_kv_e4m3(w.v_pool.to(DEV), w.block_size)
    q = w.q.to(DEV)
    tables = tables_to_device(_lists(w))
    lens = torch.from_numpy(w.seq_lens.astype(np.int32)).to(DEV)
    ws = ops.decode_workspace(q, k8)
    got = ops.decode(q, k8, v8, tables, lens, w.block_size, w.scale, ws, k_scale=ks, v_scale=vs, window=77)
    kd = po.dequantize_kv_e4m3(k8.cpu().view(torch.uint8), ks.cpu(), w.block_size)
    vd = po.dequantize_kv_e4m3(v8.cpu().view(torch.uint8), vs.cpu(), w.block_size)
    assert_close(got, po.paged_decode(w.q, kd, vd, _lists(w), w.seq_lens, w.block_size, w.scale, window=77), 6e-2,
                 "fp8 window")
    # blocks wholly before the window may hold anything, including NaN: they are never read; older keys inside
    # the window's first block are real keys of the sequence (finite) and are masked out by selection
    w = make_decode("c2", batch=2, len_range=(300, 400), seed=3)
    kp, vp = w.k_pool.clone(), w.v_pool.clone()
    window = 50
    for b in range(2):
        n = int(w.seq_lens[b])
        first_block = (n - window) // 16
        for pos in range(n - window):
            slot = int(w.block_tables[b][pos // 16]) * 16 + pos % 16
            kp[slot] = float("nan") if pos // 16 < first_block else 1.0e4
            vp[slot] = float("nan") if pos // 16 < first_block else -1.0e4
    q = w.q.to(DEV)
    tables = tables_to_device(_lists(w))
    lens = torch.from_numpy(w.seq_lens.astype(np.int32)).to(DEV)
    got = ops.decode(q, kp.to(DEV), vp.to(DEV), tables, lens, 16, w.scale, ops.decode_workspace(q, kp.to(DEV)),
                     window=window)
    want = po.paged_decode(w.q, w.k_pool, w.v_pool, _lists(w), w.seq_lens, 16, w.scale, window=window)
    assert_close(got, want, 2e-2, "poisoned keys before the window")


def test_decode_step_in_a_hip_graph():
    """The append + decode launches of one step, captured once and replayed: the entry points allocate nothing,
    clear nothing with memsets and read lengths, slots and tables from device memory, so a serving loop can
    update those buffers in place and replay.  Every replay is checked against the checker, with eager work
    and synchronisations between the replays."""
    announce("decode in a HIP graph")
    rng = np.random.default_rng(91)
    hq, hkv, d, bs, nb, batch = 8, 2, 128, 16, 64, 3
    lens = np.array([37, 5, 60], dtype=np.int32)
    tables = np.full((batch, 8), -1, dtype=np.int32)
    perm = rng.permutation(nb)
    for b in range(batch):
        tables[b, :6] = perm[b * 6 : b * 6 + 6]  # room for 96 tokens each
    kp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16)
    vp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(torch.bfloat16)
    kc, vc = kp.to(DEV), vp.to(DEV)
    q = torch.zeros(batch, hq, d, dtype=torch.bfloat16, device=DEV)
    k_new = torch.zeros(batch, hkv, d, dtype=torch.bfloat16, device=DEV)
    v_new = torch.zeros_like(k_new)
    lens_dev = torch.from_numpy(lens).to(DEV)
    slots_dev = torch.full((batch,), -1, dtype=torch.int64, device=DEV)  # the warm-up step appends nothing
    tables_dev = torch.from_numpy(tables).to(DEV)
    out = torch.empty_like(q)
    ws = ops.decode_workspace(q, kc)

    def step():
        ops.kv_scatter(kc, vc, k_new, v_new, slots_dev)
        ops.decode(q, kc, vc, tables_dev, lens_dev, bs, d ** -0.5, ws, out=out)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    k_ref, v_ref = kp.clone(), vp.clone()
    for it in range(4):
        lens += 1  # every sequence appends one token, then attends it
        qh = torch.from_numpy(rng.standard_normal((batch, hq, d)).astype(np.float32)).to(torch.bfloat16)
        kh = torch.from_numpy(rng.standard_normal((batch, hkv, d)).astype(np.float32)).to(torch.bfloat16)
        vh = torch.from_numpy(rng.standard_normal((batch, hkv, d)).astype(np.float32)).to(torch.bfloat16)
        slots = np.array([tables[b, (lens[b] - 1) // bs] * bs + (lens[b] - 1) % bs for b in range(batch)])
        q.copy_(qh.to(DEV)); k_new.copy_(kh.to(DEV)); v_new.copy_(vh.to(DEV))
        lens_dev.copy_(torch.from_numpy(lens).to(DEV)); slots_dev.copy_(torch.from_numpy(slots).to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        k_ref[slots] = kh
        v_ref[slots] = vh
        want = po.paged_decode(qh, k_ref, v_ref, [t[t >= 0].tolist() for t in tables], lens.tolist(), bs, d ** -0.5)
        assert_close(out, want, 2e-2, f"replay {it}")
        assert torch.equal(kc.cpu(), k_ref)
        (torch.ones(1000, device=DEV) * 2).sum().item()  # eager work between replays


@pytest.mark.parametrize("hq,hkv,d,kv", [
    (8, 1, 128, "bf16"),   # one kv head: a wave load covers 4 tokens, two 16-token blocks per loop iteration
    (4, 1, 128, "f16"),
    (4, 1, 64, "bf16"),    # 8 tokens per wave load: four blocks per iteration
    (6, 2, 64, "bf16"),    # two kv heads of D=64: 4 tokens per load
    (8, 1, 128, "fp8"),    # fp8 rows of 8 lanes, 8 tokens per load, two blocks per iteration
    (4, 1, 256, "fp8"),
    (8, 2, 128, "fp8"),    # 4 tokens per load: the eight steps in flight come from two blocks
    (8, 4, 128, "fp8"),    # 2 tokens per load: eight steps are one block
    (4, 2, 64, "fp8"),     # fp8 rows of 4 lanes, 8 tokens per load
    (32, 8, 128, "fp8"),   # the long-context workload's layout: one token per load, 16 steps per block
    (8, 2, 96, "bf16"),    # head sizes between the compiled ones
    (6, 2, 80, "fp8"),
    (4, 1, 192, "fp8"),
    (4, 4, 160, "f16"),
])
def test_few_kv_heads_with_blocks_of_16(hq, hkv, d, kv):
    """Layouts whose loop takes several blocks per iteration: ragged lengths around block and iteration
    boundaries, poisoned tails, a short table, a bad block id, an empty sequence, sliding windows and extra
    zero keys."""
    announce(f"decode few kv heads hq={hq} hkv={hkv} d={d} {kv}")
    rng = np.random.default_rng(400 + hq + d)
    bs, nb = 16, 160
    dtype = torch.float16 if kv == "f16" else torch.bfloat16
    lens = [1, 15, 16, 17, 31, 32, 33, 47, 48, 49, 64, 65, 127, 128, 129, 500, 0, 40, 90]
    perm = rng.permutation(nb).tolist()
    tables, at = [], 0
    for n in lens:
        c = -(-n // bs)
        tables.append(perm[at : at + c])
        at += c
    tables[-2] = tables[-2][:1]          # covers 16 of the 40 keys: the rest are zero keys
    tables[-1][-1] = 100000              # a block id outside the pool acts as a missing block
    q = torch.from_numpy(rng.standard_normal((len(lens), hq, d)).astype(np.float32)).to(dtype)
    kp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
    vp = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
    for b, n in enumerate(lens):  # poison every slot past a sequence's end inside its last block
        if n % bs and len(tables[b]) == -(-n // bs) and tables[b][-1] < nb:
            lo = tables[b][-1] * bs + n % bs
            kp[lo : (tables[b][-1] + 1) * bs] = float("nan")
            vp[lo : (tables[b][-1] + 1) * bs] = float("inf")
    want_tables = [list(t) for t in tables]
    want_tables[-1][-1] = -1
    scale = d ** -0.5
    if kv == "fp8":
        kp, vp = torch.nan_to_num(kp, nan=0.0), torch.nan_to_num(vp, posinf=0.0)  # a quantised tile holds no NaN
        kb, ks = ops.quantize_kv_e4m3(kp.to(DEV), bs)
        vb, vs = ops.quantize_kv_e4m3(vp.to(DEV), bs)
        kd = po.dequantize_kv_e4m3(kb.cpu().view(torch.uint8), ks.cpu(), bs)
        vd = po.dequantize_kv_e4m3(vb.cpu().view(torch.uint8), vs.cpu(), bs)
        pools, ref, extra, tol = (kb, vb), (kd, vd), dict(k_scale=ks, v_scale=vs), 2e-2
    else:
        pools, ref, extra, tol = (kp.to(DEV), vp.to(DEV)), (kp, vp), {}, 2e-2

    def checked(window=0, pad=False):
        kref, vref = ref
        # blocks the table does not hold are zero keys: give the checker tables cut at the first bad entry
        cut = []
        for t in want_tables:
            good = []
            for b in t:
                if b < 0:
                    break
                good.append(b)
            cut.append(good)
        return po.paged_decode(q, kref, vref, cut, lens, bs, scale, pad_zero_keys=pad, window=window)

    got = run_decode(q.to(DEV), *pools, tables, lens, bs, scale, **extra)
    assert_close(got, checked(), tol, "plain")
    assert not got[lens.index(0)].any()
    ez = [max(lens) - n for n in lens]
    got = run_decode(q.to(DEV), *pools, tables, lens, bs, scale, extra_zero=ez, **extra)
    assert_close(got, checked(pad=True), tol, "extra zero keys")
    ws = ops.decode_workspace(q.to(DEV), pools[0])
    for window in (1, 5, 16, 33, 100):
        got = ops.decode(q.to(DEV), *pools, tables_to_device(tables), torch.tensor(lens, dtype=torch.int32, device=DEV),
                         bs, scale, ws, None, extra.get("k_scale"), extra.get("v_scale"), window=window)
        assert_close(got, checked(window=window), tol, f"window {window}")
