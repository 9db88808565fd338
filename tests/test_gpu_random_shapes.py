"""Seeded random configurations of decode and chunked prefill against the checker: head layouts, head dims,
block sizes, ragged lengths, windows, fp8 pools, short tables.  Each case is small; together they walk the
dispatch space (packed / generic loops, single- and multi-block iterations, matrix-core / vector prefill)."""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import ops
from tests.gpu_helpers import DEV, announce, assert_close, tables_to_device

pytestmark = pytest.mark.gpu


def _draw(rng):
    d = int(rng.choice([32, 64, 128, 256]))
    hkv = int(rng.choice([1, 2, 3, 4, 8]))
    n_rep = int(rng.choice([1, 2, 3, 4, 7, 8, 12]))
    bs = int(rng.choice([1, 4, 8, 16, 16, 16, 32, 48]))
    kind = str(rng.choice(["bf16", "bf16", "f16", "f32", "fp8"]))
    batch = int(rng.integers(1, 7))
    return d, hkv, n_rep, bs, kind, batch


def _pool(rng, nb, bs, hkv, d, dtype):
    k = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
    v = torch.from_numpy(rng.standard_normal((nb * bs, hkv, d)).astype(np.float32)).to(dtype)
    return k, v


def _tables(rng, lens, bs, spare=2):
    need = [-(-int(n) // bs) for n in lens]
    nb = sum(need) + spare
    perm = rng.permutation(nb)
    tables, at = [], 0
    for n in need:
        tables.append(perm[at : at + n].tolist())
        at += n
    return tables, nb


@pytest.mark.parametrize("seed", range(24))
def test_random_decode(seed):
    rng = np.random.default_rng(7000 + seed)
    d, hkv, n_rep, bs, kind, batch = _draw(rng)
    hq = hkv * n_rep
    announce(f"random decode seed={seed} hq={hq} hkv={hkv} d={d} bs={bs} {kind} batch={batch}")
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32, "fp8": torch.bfloat16}[kind]
    lens = rng.integers(0, 6 * max(bs, 16) + 1, batch).tolist()
    if seed % 3 == 0:
        lens[0] = int(rng.integers(300, 700))
    tables, nb = _tables(rng, lens, bs)
    short = seed % 4 == 1 and len(tables[-1]) > 1
    if short:
        tables[-1] = tables[-1][:-1]  # the last block of the last sequence is missing: zero keys
    k, v = _pool(rng, nb, bs, hkv, d, dtype)
    q = torch.from_numpy(rng.standard_normal((batch, hq, d)).astype(np.float32)).to(dtype)
    scale = d ** -0.5
    window = int(rng.choice([0, 0, 1, 5, 40]))
    if short:
        window = 0  # zero keys and windows are separate features
    if kind == "fp8":
        if bs > 256 or d % 16:
            pytest.skip("fp8 tile limits")
        kb, ks = ops.quantize_kv_e4m3(k.to(DEV), bs)
        vb, vs = ops.quantize_kv_e4m3(v.to(DEV), bs)
        kref = po.dequantize_kv_e4m3(kb.cpu().view(torch.uint8), ks.cpu(), bs)
        vref = po.dequantize_kv_e4m3(vb.cpu().view(torch.uint8), vs.cpu(), bs)
        pools, extra, tol = (kb, vb), (ks, vs), 2e-2
    else:
        kref, vref, pools, extra = k, v, (k.to(DEV), v.to(DEV)), (None, None)
        tol = 1e-5 if kind == "f32" else 2e-2
    ws = ops.decode_workspace(q.to(DEV), pools[0])
    got = ops.decode(q.to(DEV), *pools, tables_to_device(tables), torch.tensor(lens, dtype=torch.int32, device=DEV), bs,
                     scale, ws, None, *extra, window=window)
    want = po.paged_decode(q, kref, vref, tables, lens, bs, scale, window=window)
    assert_close(got, want, tol, f"decode window={window}")


@pytest.mark.parametrize("seed", range(16))
def test_random_decode_head_sizes_between(seed):
    """Decode with head sizes between the compiled ones (multiples of 8; of 16 for fp8 pools): the next larger
    instance with the lanes past the row's end idle."""
    rng = np.random.default_rng(7100 + seed)
    _, hkv, n_rep, bs, kind, batch = _draw(rng)
    d = int(rng.choice([16, 48, 80, 96, 112, 144, 160, 192, 208, 240] if kind == "fp8" else
                       [8, 24, 40, 48, 56, 72, 80, 96, 104, 120, 136, 160, 192, 248]))
    hq = hkv * n_rep
    announce(f"random decode seed={seed} hq={hq} hkv={hkv} d={d} bs={bs} {kind} batch={batch}")
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32, "fp8": torch.bfloat16}[kind]
    lens = rng.integers(0, 6 * max(bs, 16) + 1, batch).tolist()
    if seed % 3 == 0:
        lens[0] = int(rng.integers(300, 700))
    tables, nb = _tables(rng, lens, bs)
    k, v = _pool(rng, nb, bs, hkv, d, dtype)
    q = torch.from_numpy(rng.standard_normal((batch, hq, d)).astype(np.float32)).to(dtype)
    scale = d ** -0.5
    window = int(rng.choice([0, 0, 1, 5, 40]))
    if kind == "fp8":
        if bs > 256:
            pytest.skip("fp8 tile limits")
        kb, ks = ops.quantize_kv_e4m3(k.to(DEV), bs)
        vb, vs = ops.quantize_kv_e4m3(v.to(DEV), bs)
        kref = po.dequantize_kv_e4m3(kb.cpu().view(torch.uint8), ks.cpu(), bs)
        vref = po.dequantize_kv_e4m3(vb.cpu().view(torch.uint8), vs.cpu(), bs)
        pools, extra, tol = (kb, vb), (ks, vs), 2e-2
    else:
        kref, vref, pools, extra = k, v, (k.to(DEV), v.to(DEV)), (None, None)
        tol = 1e-5 if kind == "f32" else 2e-2
    ws = ops.decode_workspace(q.to(DEV), pools[0])
    got = ops.decode(q.to(DEV), *pools, tables_to_device(tables), torch.tensor(lens, dtype=torch.int32, device=DEV), bs,
                     scale, ws, None, *extra, window=window)
    want = po.paged_decode(q, kref, vref, tables, lens, bs, scale, window=window)
    assert_close(got, want, tol, f"decode window={window}")


@pytest.mark.parametrize("seed", range(16))
def test_random_chunked_prefill(seed):
    rng = np.random.default_rng(9000 + seed)
    d, hkv, n_rep, bs, kind, batch = _draw(rng)
    if kind == "fp8":
        kind = "bf16"
    n_rep = min(n_rep, 8)
    hq = hkv * n_rep
    announce(f"random prefill seed={seed} hq={hq} hkv={hkv} d={d} bs={bs} {kind} batch={batch}")
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[kind]
    prefix = rng.integers(0, 200, batch).tolist()
    chunk = rng.integers(1, 100, batch).tolist()
    if seed % 5 == 0:
        prefix[0] = 0
    cmax = max(chunk)
    tables, nb = _tables(rng, [p + c for p, c in zip(prefix, chunk)], bs)
    k, v = _pool(rng, nb, bs, hkv, d, dtype)
    q = torch.from_numpy(rng.standard_normal((batch, cmax, hq, d)).astype(np.float32)).to(dtype)
    scale = d ** -0.5
    window = int(rng.choice([0, 0, 7, 64]))
    out = torch.zeros(batch * cmax, hq, d, dtype=dtype, device=DEV)
    i32 = lambda x: torch.tensor(list(x), dtype=torch.int32, device=DEV)
    ops.prefill_paged(q.reshape(-1, hq, d).to(DEV), k.to(DEV), v.to(DEV), tables_to_device(tables),
                      i32(p + c for p, c in zip(prefix, chunk)), i32(chunk), i32(np.arange(batch) * cmax), cmax, bs, scale,
                      out=out, window=window)
    want = po.paged_prefill_chunk(q, k, v, tables, prefix, chunk, bs, scale, window=window)
    assert_close(out.reshape(batch, cmax, hq, d), want, 1e-5 if kind == "f32" else 2e-2, f"prefill window={window}")


@pytest.mark.parametrize("seed", range(24))
def test_random_matrix_core_prefill(seed):
    """Shapes the table-driven matrix-core prefill kernels take (head_dim 32, 64 and 128: the assembly loop with and
    without lower bounds; head_dim 256), drawn at random: block sizes that are multiples of 16, ragged prefixes and
    chunks, sliding windows, per-row first keys, absent blocks.  Every case against the vector kernel (which
    states the zero-row rule of absent blocks), cases without absent blocks and first keys also against the
    checker."""
    _matrix_core_case(np.random.default_rng(9500 + seed), seed, [32, 64, 128, 128, 256])


@pytest.mark.parametrize("seed", range(16))
def test_random_matrix_core_prefill_head_sizes_between(seed):
    """The same with head sizes between the compiled ones (multiples of 8): rows in memory shorter than the
    kernel's, the reference's "any head_dim" (attention/config.py:22-24)."""
    _matrix_core_case(np.random.default_rng(9600 + seed), seed, [8, 24, 40, 48, 56, 72, 80, 96, 104, 112, 120, 160, 192, 248])


def _matrix_core_case(rng, seed, dims):
    d = int(rng.choice(dims))
    hkv = int(rng.choice([1, 2, 4]))
    n_rep = int(rng.choice([1, 2, 3, 4, 8]))
    hq = hkv * n_rep
    bs = int(rng.choice([16, 16, 32, 48, 64]))
    dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float16
    batch = int(rng.integers(1, 5))
    prefix = rng.integers(0, 1500, batch).tolist()
    chunk = rng.integers(1, 300, batch).tolist()
    if seed % 4 == 0:
        prefix[0] = 0
    window = int(rng.choice([0, 0, 20, 64, 300]))
    with_first = rng.random() < 0.4
    with_absent = rng.random() < 0.4
    announce(f"random matrix-core prefill seed={seed} hq={hq} hkv={hkv} d={d} bs={bs} {dtype} batch={batch} "
             f"window={window} first_keys={with_first} absent={with_absent}")
    cmax = max(chunk)
    tables, nb = _tables(rng, [p + c for p, c in zip(prefix, chunk)], bs)
    k, v = _pool(rng, nb, bs, hkv, d, dtype)
    if with_absent:
        for t in tables:
            for i in range(len(t)):
                if rng.random() < 0.15:
                    t[i] = -1 if rng.random() < 0.7 else nb + 3
    q = torch.from_numpy(rng.standard_normal((batch, cmax, hq, d)).astype(np.float32)).to(dtype)
    first = None
    if with_first:  # a row's document starts at a random earlier position, non-decreasing along the sequence
        rows = []
        for p, c in zip(prefix, chunk):
            starts = np.sort(rng.integers(0, p + c, max(1, (p + c) // 150)))
            pos = p + np.arange(cmax)
            f = np.zeros(cmax, dtype=np.int32)
            for st in starts:
                f = np.where(pos >= st, st, f)
            rows.append(np.minimum(f, pos).astype(np.int32))
        first = torch.from_numpy(np.stack(rows).reshape(-1)).to(DEV)
    i32 = lambda x: torch.tensor(list(x), dtype=torch.int32, device=DEV)
    args = (q.reshape(-1, hq, d).to(DEV), k.to(DEV), v.to(DEV), tables_to_device(tables),
            i32(p + c for p, c in zip(prefix, chunk)), i32(chunk), i32(np.arange(batch) * cmax), cmax, bs, d ** -0.5)
    out = torch.zeros(batch * cmax, hq, d, dtype=dtype, device=DEV)
    got = ops.prefill_paged(*args, out=out, window=window, row_first_key=first).float().cpu().reshape(batch, cmax, hq, d)
    ref = ops.prefill_paged(*args, window=window, row_first_key=first, rowwise=True).float().cpu().reshape(batch, cmax, hq, d)
    for b, c in enumerate(chunk):
        assert_close(got[b, :c], ref[b, :c], 2e-2, f"against the vector kernel, sequence {b}")
    if not with_absent and not with_first:
        want = po.paged_prefill_chunk(q, k, v, tables, prefix, chunk, bs, d ** -0.5, window=window)
        assert_close(got, want, 2e-2, "against the checker")


@pytest.mark.parametrize("seed", range(16))
def test_random_dense_prefill_of_any_length(seed):
    """Dense causal prefill the way `_prefill_attention` hands it over (flex_backend.py:144-185): a pool of B blocks
    of T rows with the identity table, T of any length (so 16-key groups run into the next sequence's rows and, at
    the end of the pool, past it), head sizes 32 / 64 / 128 / 256, with and without a sliding window; against the
    checker."""
    _dense_case(np.random.default_rng(9700 + seed), seed, [32, 64, 128, 256])


@pytest.mark.parametrize("seed", range(12))
def test_random_dense_prefill_head_sizes_between(seed):
    """The same with head sizes between the compiled ones."""
    _dense_case(np.random.default_rng(9800 + seed), seed, [8, 16, 40, 48, 72, 88, 96, 120, 136, 192, 224])


def _dense_case(rng, seed, dims):
    d = int(rng.choice(dims))
    hkv = int(rng.choice([1, 2, 4]))
    hq = hkv * int(rng.choice([1, 2, 4, 7]))
    dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float16
    b = int(rng.integers(1, 5))
    t = int(rng.choice([rng.integers(1, 40), rng.integers(40, 300), rng.integers(300, 900)]))
    window = int(rng.choice([0, 0, 13, 100]))
    announce(f"random dense prefill seed={seed} hq={hq} hkv={hkv} d={d} {dtype} batch={b} length={t} window={window}")
    q, k, v = (torch.from_numpy(rng.standard_normal((b, t, h, d)).astype(np.float32)).to(dtype) for h in (hq, hkv, hkv))
    i32 = lambda x: torch.tensor(list(x), dtype=torch.int32, device=DEV)
    ident = torch.arange(b, dtype=torch.int32, device=DEV).reshape(b, 1).contiguous()
    got = ops.prefill_paged(q.reshape(b * t, hq, d).to(DEV), k.reshape(b * t, hkv, d).to(DEV), v.reshape(b * t, hkv, d).to(DEV),
                            ident, i32([t] * b), i32([t] * b), i32(np.arange(b) * t), t, t, d ** -0.5, window=window)
    want = po.dense_prefill(q, k, v, d ** -0.5, window=window)
    assert_close(got.reshape(b, t, hq, d), want, 2e-2, "against the checker")
