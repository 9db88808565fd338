"""``pa_decode_static`` (the decode entry point that allocates nothing: its partials go to a scratch array the
library holds on the GPU) against ``pa_decode`` with a caller's workspace, through the C ABI.

Both run the same kernels on the same partition of the batch, so the outputs must be equal bit for bit.  The
scratch array keeps the previous call's contents: the second call of each test is a smaller problem, so stale
partials of the first would show up in it.
"""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import _lib, ops
from research_amd.workloads import make_decode
from tests.gpu_helpers import DEV, announce, assert_close, tables_to_device

pytestmark = pytest.mark.gpu


def _both(w, k_pool, v_pool, k_scale=None, v_scale=None, window=0):
    q = w.q.to(DEV)
    tables = tables_to_device([t.tolist() for t in w.block_tables])
    lens = torch.from_numpy(np.asarray(w.seq_lens, dtype=np.int32)).to(DEV)
    ws = ops.decode_workspace(q, k_pool)
    want = ops.decode(q, k_pool, v_pool, tables, lens, w.block_size, w.scale, ws, None, k_scale, v_scale,
                      window=window)
    out = torch.full_like(q, float("nan"))
    before = torch.cuda.memory_allocated()
    got = ops.decode_static(q, k_pool, v_pool, tables, lens, w.block_size, w.scale, None, k_scale, v_scale, out=out,
                            window=window)
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    return got, want


def test_two_calls_in_a_row_second_smaller_bf16():
    announce("decode_static bf16: 24 sequences, then 3 shorter ones")
    big = make_decode("c4", batch=24, len_range=(64, 6000))
    got, want = _both(big, big.k_pool.to(DEV), big.v_pool.to(DEV))
    assert torch.equal(got, want)
    ref = po.paged_decode(big.q, big.k_pool, big.v_pool, [t.tolist() for t in big.block_tables], big.seq_lens,
                          big.block_size, big.scale)
    assert_close(got, ref, 2e-2, "static scratch, first call")
    small = make_decode("c4", batch=3, len_range=(64, 900), seed=5)
    got, want = _both(small, small.k_pool.to(DEV), small.v_pool.to(DEV))
    assert torch.equal(got, want)
    ref = po.paged_decode(small.q, small.k_pool, small.v_pool, [t.tolist() for t in small.block_tables],
                          small.seq_lens, small.block_size, small.scale)
    assert_close(got, ref, 2e-2, "static scratch, second (smaller) call")


def test_two_calls_in_a_row_fp32_and_fp8():
    announce("decode_static fp32 c1, then one long fp8 sequence, then a short one")
    w = make_decode("c1")
    got, want = _both(w, w.k_pool.to(DEV), w.v_pool.to(DEV))
    assert torch.equal(got, want)
    long = make_decode("c5", batch=1, len_range=(20000, 20001))
    k8, ks = ops.quantize_kv_e4m3(long.k_pool.to(DEV), long.block_size)
    v8, vs = ops.quantize_kv_e4m3(long.v_pool.to(DEV), long.block_size)
    got, want = _both(long, k8, v8, ks, vs)
    assert torch.equal(got, want)
    short = make_decode("c5", batch=2, len_range=(100, 400), seed=9)
    k8, ks = ops.quantize_kv_e4m3(short.k_pool.to(DEV), short.block_size)
    v8, vs = ops.quantize_kv_e4m3(short.v_pool.to(DEV), short.block_size)
    got, want = _both(short, k8, v8, ks, vs, window=128)
    assert torch.equal(got, want)


def test_shapes_beyond_the_scratch_are_rejected_before_any_launch():
    announce("decode_static: batch 8192 is refused")
    q = torch.zeros((8192, 32, 128), dtype=torch.bfloat16, device=DEV)
    pool = torch.zeros((16, 8, 128), dtype=torch.bfloat16, device=DEV)
    tables = torch.full((8192, 1), -1, dtype=torch.int32, device=DEV)
    lens = torch.zeros(8192, dtype=torch.int32, device=DEV)
    with pytest.raises(_lib.PagedAttnError, match="scratch") as e:
        ops.decode_static(q, pool, pool, tables, lens, 16, 1.0)
    assert e.value.status == _lib.PA_ERR_WORKSPACE
