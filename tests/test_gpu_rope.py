"""Rotary embedding fused with the KV append on the GPU: bit-exact against the elementwise statement
evaluated with torch on the CPU (the checker's rope_literal), for both table layouts, all three types, the
fp8 pool, and through the backend."""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import ops
from research_amd.inference import CacheConfig, HipPagedAttentionBackend, InferenceContext
from tests.gpu_helpers import DEV, announce, assert_close

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


def _case(dtype, n, hq, hkv, d, seed, max_pos=500):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n, hq, d, generator=g).to(dtype)
    k = torch.randn(n, hkv, d, generator=g).to(dtype)
    v = torch.randn(n, hkv, d, generator=g).to(dtype)
    pos = torch.randint(0, max_pos, (n,), generator=g)
    return q, k, v, pos


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (4, 4, 64), (6, 1, 32), (2, 2, 256)])
def test_rope_append_bit_exact(dtype, hq, hkv, d):
    announce(f"rope append {dtype} hq={hq} hkv={hkv} d={d}")
    n, bs, nb = 75, 16, 12
    q, k, v, pos = _case(dtype, n, hq, hkv, d, seed=7 + d)
    cos, sin = (t[0] for t in po.rope_tables(pos[None], d, 10000.0, dtype))  # one row per token
    want_q, want_k = po.rope_literal(q, cos, sin), po.rope_literal(k, cos, sin)
    slots = torch.randperm(nb * bs, generator=torch.Generator().manual_seed(3))[:n]
    slots[5] = -1
    slots[40] = nb * bs + 3  # past the pool: skipped like a negative slot
    kc = torch.full((nb * bs, hkv, d), 7.0, dtype=dtype, device=DEV)
    vc = torch.full_like(kc, 7.0)
    k_out = torch.zeros(n, hkv, d, dtype=dtype, device=DEV)
    q_dev = q.to(DEV)
    q_rot = ops.rope_kv_append(q_dev, k.to(DEV), v.to(DEV), cos.to(DEV), sin.to(DEV), kc, vc, slots.to(DEV),
                               q_out=torch.empty_like(q_dev), k_out=k_out)
    assert torch.equal(_bits(q_rot.cpu()), _bits(want_q)) and torch.equal(q_dev.cpu(), q)  # q itself untouched
    assert torch.equal(_bits(k_out.cpu()), _bits(want_k))
    want_kc = torch.full((nb * bs, hkv, d), 7.0, dtype=dtype)
    want_vc = torch.full_like(want_kc, 7.0)
    ok = (slots >= 0) & (slots < nb * bs)
    want_kc[slots[ok]] = want_k[ok]
    want_vc[slots[ok]] = v[ok]
    assert torch.equal(_bits(kc.cpu()), _bits(want_kc)) and torch.equal(_bits(vc.cpu()), _bits(want_vc))
    # a table indexed by position, q rotated in place, no dense K copy
    table_cos, table_sin = (t[0] for t in po.rope_tables(torch.arange(500)[None], d, 10000.0, dtype))
    kc.fill_(7.0)
    vc.fill_(7.0)
    q_in = q.to(DEV)
    out = ops.rope_kv_append(q_in, k.to(DEV), v.to(DEV), table_cos.to(DEV), table_sin.to(DEV), kc, vc, slots.to(DEV),
                             positions=pos.to(torch.int32).to(DEV))
    assert out.data_ptr() == q_in.data_ptr() and torch.equal(_bits(q_in.cpu()), _bits(want_q))
    assert torch.equal(_bits(kc.cpu()), _bits(want_kc)) and torch.equal(_bits(vc.cpu()), _bits(want_vc))
    # no cache at all: rotation only
    k_out.zero_()
    ops.rope_kv_append(q.to(DEV), k.to(DEV), v.to(DEV), cos.to(DEV), sin.to(DEV), None, None, None, k_out=k_out)
    assert torch.equal(_bits(k_out.cpu()), _bits(want_k))


def test_rope_append_matches_the_exact_rotation():
    """Independent of torch's elementwise statement: complex multiplication in float64."""
    announce("rope vs complex rotation")
    n, hq, hkv, d = 33, 4, 2, 64
    q, k, v, pos = _case(torch.float32, n, hq, hkv, d, seed=21, max_pos=90)
    cos, sin = (t[0] for t in po.rope_tables(pos[None], d, 10000.0, torch.float32))
    angle = pos.numpy()[:, None].astype(np.float64) * 10000.0 ** (-np.arange(0, d, 2, dtype=np.float64) / d)
    k_out = torch.zeros(n, hkv, d, device=DEV)
    q_rot = ops.rope_kv_append(q.to(DEV), k.to(DEV), v.to(DEV), cos.to(DEV), sin.to(DEV), None, None, None, k_out=k_out)
    assert_close(q_rot, po.rope_exact(q, angle), 2e-5, "q")
    assert_close(k_out, po.rope_exact(k, angle), 2e-5, "k")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rope_append_into_an_fp8_pool(dtype):
    """Equals rotating on the CPU and appending the rotated rows with the checker's append policy, bytes and
    scales, over two calls (prefill of ragged lengths, then one more token each)."""
    announce(f"rope append fp8 {dtype}")
    hq, hkv, d, bs, nb = 8, 2, 128, 16, 10
    g = torch.Generator().manual_seed(31)
    lens = [37, 16, 5]
    tables = [[3, 7, 1], [0], [9]]
    bits_k = torch.zeros(nb * bs, hkv, d, dtype=torch.uint8)
    bits_v = torch.zeros_like(bits_k)
    sc_k = torch.ones(nb, hkv)
    sc_v = torch.ones(nb, hkv)
    kc = bits_k.clone().view(torch.float8_e4m3fn).to(DEV)
    vc = bits_v.clone().view(torch.float8_e4m3fn).to(DEV)
    ksc, vsc = sc_k.clone().to(DEV), sc_v.clone().to(DEV)
    table_cos, table_sin = (t[0] for t in po.rope_tables(torch.arange(64)[None], d, 10000.0, dtype))
    for step in range(2):
        if step == 0:
            pos = torch.cat([torch.arange(n) for n in lens])
            slots = torch.tensor([tables[b][p // bs] * bs + p % bs for b, n in enumerate(lens) for p in range(n)])
        else:
            pos = torch.tensor(lens)
            tables[1].append(5)  # sequence 1 filled its block
            slots = torch.tensor([tables[b][n // bs] * bs + n % bs for b, n in enumerate(lens)])
        n = len(pos)
        q = torch.randn(n, hq, d, generator=g).to(dtype)
        k = (torch.randn(n, hkv, d, generator=g) * (1 + step * 3)).to(dtype)  # later rows raise the scales
        v = torch.randn(n, hkv, d, generator=g).to(dtype)
        cos, sin = table_cos[pos], table_sin[pos]
        want_q, want_k = po.rope_literal(q, cos, sin), po.rope_literal(k, cos, sin)
        po.append_kv_e4m3(bits_k, sc_k, want_k, slots.tolist(), bs)
        po.append_kv_e4m3(bits_v, sc_v, v, slots.tolist(), bs)
        q_rot = ops.rope_kv_append_e4m3(q.to(DEV), k.to(DEV), v.to(DEV), table_cos.to(DEV), table_sin.to(DEV), kc, vc,
                                        ksc, vsc, slots.to(DEV), bs, positions=pos.to(torch.int32).to(DEV),
                                        q_out=torch.empty(n, hq, d, dtype=dtype, device=DEV))
        assert torch.equal(_bits(q_rot.cpu()), _bits(want_q))
        assert torch.equal(kc.cpu().view(torch.uint8), bits_k) and torch.equal(vc.cpu().view(torch.uint8), bits_v)
        assert torch.equal(ksc.cpu(), sc_k) and torch.equal(vsc.cpu(), sc_v)


def test_forward_rope_through_the_backend():
    """forward_rope == apply the rotation, then forward: dense prefill, chunked prefill and decode."""
    from research_amd.inference import PagedKVCache, allocate_and_build_context, extend_and_build_context

    announce("backend forward_rope")
    g = torch.Generator().manual_seed(61)
    hq, hkv, d, bs = 8, 2, 64, 16
    config = CacheConfig(num_layers=2, num_kv_heads=hkv, head_dim=d, num_blocks=8, block_size=bs, device="cuda")
    fused, plain = HipPagedAttentionBackend(config), HipPagedAttentionBackend(config)
    for be in (fused, plain):
        be.set_num_heads(hq)
    caches = [PagedKVCache(8, bs), PagedKVCache(8, bs)]
    n = 21
    q = torch.randn(1, n, hq, d, generator=g).to(torch.bfloat16)
    k = torch.randn(1, n, hkv, d, generator=g).to(torch.bfloat16)
    v = torch.randn(1, n, hkv, d, generator=g).to(torch.bfloat16)
    table_cos, table_sin = (t[0] for t in po.rope_tables(torch.arange(64)[None], d, 10000.0, torch.bfloat16))
    cos, sin = table_cos[:n], table_sin[:n]
    q_r = po.rope_literal(q[0], cos, sin)[None]
    k_r = po.rope_literal(k[0], cos, sin)[None]
    ctx_f, _ = allocate_and_build_context(caches[0], seq_id=0, token_ids=list(range(n)))
    ctx_p, _ = allocate_and_build_context(caches[1], seq_id=0, token_ids=list(range(n)))
    out_f = fused.forward_rope(q.cuda(), k.cuda(), v.cuda(), cos[None].cuda(), sin[None].cuda(), 1, ctx_f)
    out_p = plain.forward(q_r.cuda(), k_r.cuda(), v.cuda(), 1, ctx_p)
    assert torch.equal(out_f, out_p)
    assert torch.equal(fused.k_cache, plain.k_cache) and torch.equal(fused.v_cache, plain.v_cache)
    assert_close(out_f, po.dense_prefill(q_r, k_r, v, fused.scale), 2e-2, "prefill on rotated q, k")
    # decode with a position table
    q1 = torch.randn(1, 1, hq, d, generator=g).to(torch.bfloat16)
    k1 = torch.randn(1, 1, hkv, d, generator=g).to(torch.bfloat16)
    v1 = torch.randn(1, 1, hkv, d, generator=g).to(torch.bfloat16)
    ctx_f = extend_and_build_context(caches[0], seq_id=0, new_token=99, current_len=n)
    ctx_p = extend_and_build_context(caches[1], seq_id=0, new_token=99, current_len=n)
    out_f = fused.forward_rope(q1.cuda(), k1.cuda(), v1.cuda(), table_cos.cuda(), table_sin.cuda(), 1, ctx_f,
                               positions=torch.tensor([[n]]))
    q1_r = po.rope_literal(q1[0], table_cos[n : n + 1], table_sin[n : n + 1])[None]
    k1_r = po.rope_literal(k1[0], table_cos[n : n + 1], table_sin[n : n + 1])[None]
    out_p = plain.forward(q1_r.cuda(), k1_r.cuda(), v1.cuda(), 1, ctx_p)
    assert torch.equal(out_f, out_p) and torch.equal(fused.k_cache, plain.k_cache)


def test_rope_append_at_full_size():
    """The append of workload c3 (8 192 tokens, 32 q heads, 8 kv heads, D=128, positions 2048..2303 from a table)
    and a decode-step append of workload c4's shape (256 tokens at positions up to 32 767): every output bit
    against the elementwise statement on the CPU."""
    announce("rope append, c3 / c4 sizes")
    hq, hkv, d, bs = 32, 8, 128, 16
    for n, max_pos, nb, seed in ((8192, 2304, 640, 1), (256, 32768, 4096, 2)):
        g = torch.Generator().manual_seed(seed)
        q = torch.randn(n, hq, d, generator=g).to(torch.bfloat16)
        k = torch.randn(n, hkv, d, generator=g).to(torch.bfloat16)
        v = torch.randn(n, hkv, d, generator=g).to(torch.bfloat16)
        pos = torch.randint(max(0, max_pos - 256), max_pos, (n,), generator=g)
        cos_t, sin_t = (t[0] for t in po.rope_tables(torch.arange(max_pos)[None], d, 10000.0, torch.bfloat16))
        slots = torch.randperm(nb * bs, generator=g)[:n]
        kc = torch.zeros(nb * bs, hkv, d, dtype=torch.bfloat16, device=DEV)
        vc = torch.zeros_like(kc)
        q_rot = ops.rope_kv_append(q.to(DEV), k.to(DEV), v.to(DEV), cos_t.to(DEV), sin_t.to(DEV), kc, vc, slots.to(DEV),
                                   positions=pos.to(torch.int32).to(DEV), q_out=torch.empty(n, hq, d, dtype=torch.bfloat16, device=DEV))
        want_q = po.rope_literal(q, cos_t[pos], sin_t[pos])
        want_k = po.rope_literal(k, cos_t[pos], sin_t[pos])
        assert torch.equal(_bits(q_rot.cpu()), _bits(want_q))
        assert torch.equal(_bits(kc.cpu()[slots]), _bits(want_k)) and torch.equal(_bits(vc.cpu()[slots]), _bits(v))
        untouched = torch.ones(nb * bs, dtype=torch.bool)
        untouched[slots] = False
        assert not kc.cpu()[untouched].any() and not vc.cpu()[untouched].any()


def test_forward_rope_dense_prefill_into_an_fp8_pool():
    """Dense prefill attends the step's own rotated K/V (bf16) while the rows are appended to the fp8 pool."""
    from research_amd.inference import PagedKVCache, allocate_and_build_context

    announce("backend forward_rope, dense prefill, fp8 pool")
    g = torch.Generator().manual_seed(62)
    hq, hkv, d, bs = 8, 2, 64, 16
    config = CacheConfig(num_layers=1, num_kv_heads=hkv, head_dim=d, num_blocks=8, block_size=bs, device="cuda",
                         kv_format="fp8_e4m3")
    backend = HipPagedAttentionBackend(config)
    backend.set_num_heads(hq)
    n = 37
    q, k, v = (torch.randn(1, n, h, d, generator=g).to(torch.bfloat16) for h in (hq, hkv, hkv))
    cos, sin = (t[0] for t in po.rope_tables(torch.arange(n)[None], d, 10000.0, torch.bfloat16))
    ctx, _ = allocate_and_build_context(PagedKVCache(8, bs), seq_id=0, token_ids=list(range(n)))
    out = backend.forward_rope(q.cuda(), k.cuda(), v.cuda(), cos[None].cuda(), sin[None].cuda(), 0, ctx)
    q_r, k_r = po.rope_literal(q[0], cos, sin)[None], po.rope_literal(k[0], cos, sin)[None]
    assert_close(out, po.dense_prefill(q_r, k_r, v, backend.scale), 2e-2, "dense prefill")
    bits_k = torch.zeros(8 * bs, hkv, d, dtype=torch.uint8)
    bits_v = torch.zeros_like(bits_k)
    sc_k, sc_v = torch.ones(8, hkv), torch.ones(8, hkv)
    po.append_kv_e4m3(bits_k, sc_k, k_r[0], ctx.slot_mapping, bs)
    po.append_kv_e4m3(bits_v, sc_v, v[0], ctx.slot_mapping, bs)
    assert torch.equal(backend.k_cache[0].cpu().view(torch.uint8), bits_k) and torch.equal(backend.k_scale[0].cpu(), sc_k)
    assert torch.equal(backend.v_cache[0].cpu().view(torch.uint8), bits_v) and torch.equal(backend.v_scale[0].cpu(), sc_v)
