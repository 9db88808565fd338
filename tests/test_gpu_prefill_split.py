"""Chunked prefill with its keys split over workgroups (``pa_prefill_paged_ws``): launches of few query rows, whose
workgroups' tiles are cut into pieces that leave partial results in a workspace for a merge kernel.

Every case is checked against the CPU checker (2e-2, the bar of the unsplit kernels) and against
``pa_prefill_paged`` on the same inputs (6e-3: the pieces round their probabilities to 16 bits relative to
maxima of their own, so results differ by an ulp or two of the 16-bit output).  The number of pieces
follows the shapes (few workgroups, wide block tables) and is capped here by the size of the workspace handed
over: 2, 3 and 8 pieces.
"""

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import _lib, ops
from tests.gpu_helpers import DEV, announce, assert_close

pytestmark = pytest.mark.gpu


def _i32(x):
    return torch.tensor(list(x), dtype=torch.int32, device=DEV)


class Case:
    """Ragged sequences over a pool of blocks in random order; the tables are padded wide (with -1) so that the
    library sizes its split for long contexts."""

    def __init__(self, prefix, chunk, hq, hkv, d, dtype=torch.bfloat16, bs=16, seed=0, width=1024, absent=()):
        rng = np.random.default_rng(seed)
        self.prefix, self.chunk, self.bs, self.hq, self.hkv, self.d = list(prefix), list(chunk), bs, hq, hkv, d
        n = len(prefix)
        ctx = [p + c for p, c in zip(prefix, chunk)]
        need = sum(-(-t // bs) for t in ctx)
        perm = rng.permutation(need + 3)
        self.tables, at = [], 0
        for t in ctx:
            k = -(-t // bs)
            self.tables.append(perm[at: at + k].tolist())
            at += k
        for seq, blk in absent:  # absent blocks: all-zero keys
            self.tables[seq][blk] = -1
        draw = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(dtype)
        self.cmax = max(chunk)
        self.q = draw(n, self.cmax, hq, d)
        self.k = draw((need + 3) * bs, hkv, d)
        self.v = draw((need + 3) * bs, hkv, d)
        self.scale = d ** -0.5
        wide = np.full((n, max(width, max(len(t) for t in self.tables))), -1, dtype=np.int32)
        for i, t in enumerate(self.tables):
            wide[i, : len(t)] = t
        self.dev_tables = torch.from_numpy(wide).to(DEV)
        self.ctx = ctx

    def run(self, pieces=None, window=0, row_first_key=None):
        """pieces None: pa_prefill_paged; else pa_prefill_paged_ws with a workspace that holds that many pieces."""
        n = len(self.ctx)
        q = self.q.reshape(n * self.cmax, self.hq, self.d).to(DEV)
        ws = None
        if pieces is not None:
            want = ops.prefill_workspace_bytes(q, self.dev_tables, self.cmax, self.bs, self.hkv, window)
            d_rows = next(x for x in (32, 64, 128, 256) if x >= self.d)  # partial rows have the kernel's head size
            per_piece = n * self.cmax * self.hq * (d_rows + 2) * 4
            assert want >= pieces * per_piece, f"the library would cut this launch into {want // per_piece} pieces only"
            ws = torch.full((pieces * per_piece,), 0xFF, dtype=torch.uint8, device=DEV)  # NaN patterns: nothing is assumed
        out = torch.zeros_like(q)
        ops.prefill_paged(q, self.k.to(DEV), self.v.to(DEV), self.dev_tables, _i32(self.ctx), _i32(self.chunk),
                          _i32(np.arange(n) * self.cmax), self.cmax, self.bs, self.scale, out=out, window=window,
                          row_first_key=row_first_key, workspace=ws)
        return out.reshape(n, self.cmax, self.hq, self.d)

    def want(self, window=0):
        tables = [[b if b >= 0 else 0 for b in t] for t in self.tables]
        k, v = self.k.clone(), self.v.clone()
        return po.paged_prefill_chunk(self.q, k, v, tables, self.prefix, self.chunk, self.bs, self.scale, window=window)


@pytest.mark.parametrize("pieces", [2, 3, 8])
@pytest.mark.parametrize("d,hq,hkv,dtype", [(128, 8, 2, torch.bfloat16), (64, 4, 1, torch.float16),
                                           (32, 4, 2, torch.bfloat16), (256, 4, 2, torch.bfloat16),
                                           (256, 2, 1, torch.float16), (96, 8, 2, torch.bfloat16),
                                           (192, 4, 2, torch.float16), (40, 4, 1, torch.bfloat16)])
def test_one_long_sequence_in_pieces(pieces, d, hq, hkv, dtype):
    announce(f"split prefill: one sequence, {pieces} pieces, d={d} {dtype}")
    c = Case([2900], [150], hq, hkv, d, dtype=dtype, seed=pieces + d)
    base = c.run()
    got = c.run(pieces)
    assert_close(got, c.want(), 2e-2, "split vs checker")
    assert_close(got, base, 6e-3, "split vs one workgroup per group")


def test_ragged_batch_short_contexts_and_empty_pieces():
    """Contexts of a few tiles cut into 8: most pieces are empty for some workgroup; a sequence with a shorter
    chunk than the batch's longest, a dense one (no prefix: early rows see none of the later pieces' keys)."""
    announce("split prefill: ragged batch, empty pieces")
    c = Case([0, 70, 700], [130, 33, 96], 8, 2, 128, seed=5)
    base, got = c.run(), c.run(8)
    want = c.want()
    for b, n in enumerate(c.chunk):
        assert_close(got[b, :n], want[b, :n], 2e-2, f"sequence {b} vs checker")
        assert_close(got[b, :n], base[b, :n], 6e-3, f"sequence {b} vs unsplit")
        assert not got[b, n:].any()  # rows past the chunk are not written


def test_windows_first_keys_and_absent_blocks_in_pieces():
    announce("split prefill: window, per-row first keys, absent blocks")
    # (under a window a workgroup sees window + 256 keys at most: the library splits only wide windows)
    w = Case([6000, 5000], [100, 100], 8, 2, 128, seed=8)
    got = w.run(2, window=4000)
    assert_close(got, w.run(window=4000), 6e-3, "window 4000: split vs unsplit")
    assert_close(got, w.want(window=4000), 2e-2, "window 4000: split vs checker")
    c = Case([1500, 900], [100, 100], 8, 2, 128, seed=9, absent=[(0, 7), (1, 20)])
    # absent blocks are zero keys (logit 0, zero value): the checker reads a zeroed block in their place
    zk, zv = c.k.clone(), c.v.clone()
    tables = [list(t) for t in c.tables]
    spare = min(set(range(c.k.shape[0] // 16)) - {b for t in c.tables for b in t})  # a block no table names
    for t in tables:
        for i, b in enumerate(t):
            if b < 0:
                t[i] = spare
    zk[spare * 16: spare * 16 + 16] = 0
    zv[spare * 16: spare * 16 + 16] = 0
    want = po.paged_prefill_chunk(c.q, zk, zv, tables, c.prefix, c.chunk, 16, c.scale)
    assert_close(c.run(4), want, 2e-2, "absent blocks: split vs checker")
    first = np.concatenate([np.minimum(np.arange(100) + p, (np.arange(100) + p) // 300 * 300) for p in c.prefix])
    rfk = torch.from_numpy(first.astype(np.int32)).to(DEV)
    assert_close(c.run(3, row_first_key=rfk), c.run(row_first_key=rfk), 6e-3, "per-row first keys: split vs unsplit")


def test_context_longer_than_the_kernel_tables_in_pieces():
    """More keys than the kernel's LDS slot tables hold (the instance that refills them), cut into pieces; against
    the unsplit launch (the checker would take minutes on 0.11 M keys)."""
    announce("split prefill: 110 000 cached keys")
    c = Case([110000], [64], 4, 1, 128, seed=3, width=7000)
    assert_close(c.run(8), c.run(), 6e-3, "long context: split vs unsplit")


def test_workspace_rules():
    c = Case([2900], [150], 8, 2, 128, seed=1)
    q = c.q.reshape(150, 8, 128).to(DEV)
    # a launch that fills the device needs no workspace; fp32 has no split kernel; a head size between the compiled
    # ones is sized for partial rows of the next larger one
    big = torch.zeros((64, 1024), dtype=torch.int32, device=DEV)
    assert ops.prefill_workspace_bytes(torch.empty((64 * 256, 32, 128), dtype=torch.bfloat16, device=DEV), big, 256, 16, 8) == 0
    assert ops.prefill_workspace_bytes(q.float(), c.dev_tables, 150, 16, 2) == 0
    assert (ops.prefill_workspace_bytes(torch.empty((150, 8, 96), dtype=torch.bfloat16, device=DEV), c.dev_tables, 150, 16, 2)
            == ops.prefill_workspace_bytes(q, c.dev_tables, 150, 16, 2) > 0)
    # narrow tables (short contexts at most): no split either
    assert ops.prefill_workspace_bytes(q, c.dev_tables[:, :64].contiguous(), 150, 16, 2) == 0
    # a workspace too small for two pieces: the call is the unsplit one
    tiny = torch.empty(1024, dtype=torch.uint8, device=DEV)
    out = ops.prefill_paged(q, c.k.to(DEV), c.v.to(DEV), c.dev_tables, _i32(c.ctx), _i32(c.chunk), _i32([0]), 150, 16,
                            c.scale, workspace=tiny)
    assert torch.equal(out.reshape(1, 150, 8, 128), c.run())
    with pytest.raises(_lib.PagedAttnError, match="256-byte aligned"):
        ws = torch.empty(8 * 150 * 8 * 130 * 4 + 16, dtype=torch.uint8, device=DEV)[16:]
        ops.prefill_paged(q, c.k.to(DEV), c.v.to(DEV), c.dev_tables, _i32(c.ctx), _i32(c.chunk), _i32([0]), 150, 16,
                          c.scale, workspace=ws)
