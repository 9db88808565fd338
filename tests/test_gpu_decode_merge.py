"""Decode batches whose split pass merges a sequence's pieces itself, inside its one launch.

With about 128 sequences or more (``pa_decode_passes`` == 1) a workgroup that finishes a piece of a sequence counts
itself on the sequence's ticket, and the workgroup whose piece completes the sequence (or a group of its pieces, when
there are many) reads the pieces back and merges them.  Each case here is checked three ways: against the CPU checker (2e-2 for 16-bit pools, 1e-5 for
fp32, 6e-2 for fp8 against dequantise-then-attend), against ``pa_decode_split`` + ``pa_decode_reduce`` on the same
inputs (the same partials merged by the second launch, in another order: 1e-3), and for rows that must be exactly
zero.  The graph tests replay a captured append + decode step of 256 sequences with lengths, slots and queries
rewritten in place and eager calls sharing the workspace between the replays.
"""

import time

import numpy as np
import pytest
import torch

from oracle import paged_oracle as po
from research_amd import _lib, ops
from tests.gpu_helpers import DEV, announce, assert_close, tables_to_device

pytestmark = pytest.mark.gpu

DT = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32, "fp8": torch.bfloat16}


class Batch:
    """A ragged batch over a pool of 16-token blocks: tables are consecutive slices of a seeded permutation."""

    def __init__(self, lens, hq, hkv, d, kv, seed, bs=16, spare_blocks=4):
        rng = np.random.default_rng(seed)
        self.bs, self.hq, self.hkv, self.d, self.kv = bs, hq, hkv, d, kv
        self.lens = [int(n) for n in lens]
        need = sum(-(-n // bs) for n in self.lens)
        self.num_blocks = need + spare_blocks
        perm = rng.permutation(self.num_blocks)
        self.tables, at = [], 0
        for n in self.lens:
            c = -(-n // bs)
            self.tables.append(perm[at: at + c].tolist())
            at += c
        dtype = DT[kv]
        draw = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(dtype)
        self.q = draw(len(self.lens), hq, d)
        self.k = draw(self.num_blocks * bs, hkv, d)
        self.v = draw(self.num_blocks * bs, hkv, d)
        self.scale = d ** -0.5
        self.tol = {"f32": 1e-5, "fp8": 6e-2}.get(kv, 2e-2)

    def device_pools(self):
        """(k, v, k_scale, v_scale) on the device and the pools the checker reads."""
        if self.kv == "fp8":
            kb, ks = ops.quantize_kv_e4m3(self.k.to(DEV), self.bs)
            vb, vs = ops.quantize_kv_e4m3(self.v.to(DEV), self.bs)
            kd = po.dequantize_kv_e4m3(kb.cpu().view(torch.uint8), ks.cpu(), self.bs)
            vd = po.dequantize_kv_e4m3(vb.cpu().view(torch.uint8), vs.cpu(), self.bs)
            return (kb, vb, ks, vs), (kd, vd)
        return (self.k.to(DEV), self.v.to(DEV), None, None), (self.k, self.v)


def _passes(batch, hq, hkv, d, kv_dtype):
    return int(_lib.load().pa_decode_passes(batch, hq, hkv, d, ops.PA_DTYPE[kv_dtype]))


def _three_ways(b, window=0, extra_zero=None, checker_tables=None, what=""):
    """pa_decode (one launch) against the checker and against the two separate passes."""
    (kp, vp, ks, vs), (kref, vref) = b.device_pools()
    q = b.q.to(DEV)
    assert _passes(len(b.lens), b.hq, b.hkv, b.d, kp.dtype) == 1, "this batch was meant to merge inside the split pass"
    tables = tables_to_device(b.tables)
    lens = torch.tensor(b.lens, dtype=torch.int32, device=DEV)
    ez = None if extra_zero is None else torch.tensor(extra_zero, dtype=torch.int32, device=DEV)
    ws = ops.decode_workspace(q, kp)
    got = ops.decode(q, kp, vp, tables, lens, b.bs, b.scale, ws, ez, ks, vs, window=window)
    ws2 = ops.decode_workspace(q, kp)
    two = torch.full_like(q, float("nan"))
    ops.decode(q, kp, vp, tables, lens, b.bs, b.scale, ws2, ez, ks, vs, out=two, entry="pa_decode_split", window=window)
    ops.decode(q, kp, vp, tables, lens, b.bs, b.scale, ws2, ez, ks, vs, out=two, entry="pa_decode_reduce", window=window)
    torch.cuda.synchronize()
    want = po.paged_decode(b.q, kref, vref, checker_tables or b.tables, b.lens, b.bs, b.scale,
                           pad_zero_keys=extra_zero is not None, window=window)
    assert_close(got, want, b.tol, f"{what}: one launch vs checker")
    assert_close(got, two, 1e-3 if b.kv != "f32" else 1e-5, f"{what}: one launch vs split + reduce")
    # a second call on the same workspace (the tickets of the first are left counting zero)
    again = ops.decode(q, kp, vp, tables, lens, b.bs, b.scale, ws, ez, ks, vs, window=window)
    assert torch.equal(again, got), f"{what}: second call on the same workspace differs"
    return got


def _ragged(rng, batch, lo, hi, empties=0):
    lens = rng.integers(lo, hi + 1, batch)
    if empties:
        lens[rng.choice(batch, empties, replace=False)] = 0
    return lens


@pytest.mark.parametrize("batch,kv,hq,hkv,d", [
    (128, "bf16", 32, 8, 128),
    (256, "bf16", 32, 8, 128),
    (513, "bf16", 32, 8, 128),
    (2000, "bf16", 16, 8, 128),
    (256, "f16", 32, 8, 128),
    (256, "f32", 8, 2, 64),     # the generic fp32 loop
    (300, "fp8", 32, 8, 128),
    (256, "bf16", 14, 2, 64),   # Qwen2.5-0.5B's heads: a group of 7 padded to 8, one plane
    (384, "bf16", 16, 8, 256),
])
def test_ragged_batches_merge_inside_the_split_pass(batch, kv, hq, hkv, d):
    announce(f"decode merge-in-split batch={batch} {kv} hq={hq} hkv={hkv} d={d}")
    rng = np.random.default_rng(batch * 7 + d)
    lens = _ragged(rng, batch, 1, 400 if batch <= 600 else 120, empties=max(1, batch // 50))
    b = Batch(lens, hq, hkv, d, kv, seed=batch + d)
    got = _three_ways(b, what=f"B={batch} {kv}")
    for i, n in enumerate(b.lens):
        if n == 0:
            assert not got[i].any(), f"empty sequence {i} is not all zero"


@pytest.mark.parametrize("kv", ["bf16", "fp8", "f32"])
def test_window_extra_zero_keys_short_table_and_bad_block_ids(kv):
    """Every feature of the decode call in a batch that takes the one-launch path."""
    announce(f"decode merge-in-split features {kv}")
    rng = np.random.default_rng(17)
    batch = 260
    hq, hkv, d = (8, 2, 64) if kv == "f32" else (32, 8, 128)
    lens = _ragged(rng, batch, 1, 300, empties=5)
    lens[7], lens[100] = 90, 200
    b = Batch(lens, hq, hkv, d, kv, seed=5)
    checker_tables = [list(t) for t in b.tables]
    b.tables[7] = b.tables[7][:2]                    # covers 32 of the 90 keys: the rest are zero keys
    checker_tables[7] = checker_tables[7][:2]
    b.tables[100][5] = 10 ** 6                       # an id outside the pool acts as a missing block from there on
    b.tables[100][6] = -7
    checker_tables[100] = checker_tables[100][:5]
    # the checker treats everything past a short table as zero keys; the kernel treats each bad entry alone as
    # missing, so put zero keys behind the first bad entry by cutting the real table there as well
    b.tables[100] = b.tables[100][:7]
    _three_ways(b, checker_tables=checker_tables, what="short table / bad ids")
    _three_ways(b, extra_zero=[max(b.lens) - n for n in b.lens], checker_tables=checker_tables, what="extra zero keys")
    for window in (1, 16, 37, 150):
        _three_ways(b, window=window, checker_tables=checker_tables, what=f"window {window}")


def test_one_very_long_sequence_among_255_short_ones():
    """The long sequence's hundreds of pieces are merged by the one workgroup that delivers the last of them."""
    announce("decode merge-in-split: one 60 000-key sequence among 255 short ones")
    rng = np.random.default_rng(3)
    lens = _ragged(rng, 256, 16, 200)
    lens[77] = 60000
    b = Batch(lens, 32, 8, 128, "bf16", seed=11)
    _three_ways(b, what="one long sequence")
    (kp, vp, _, _), _ = b.device_pools()
    q = b.q.to(DEV)
    tables = tables_to_device(b.tables)
    dl = torch.tensor(b.lens, dtype=torch.int32, device=DEV)
    ws, out = ops.decode_workspace(q, kp), torch.empty_like(q)
    timings = {}
    for entry in ("pa_decode", "two"):
        for it in range(6):
            if it == 1:
                torch.cuda.synchronize()
                t0 = time.perf_counter()
            if entry == "two":
                ops.decode(q, kp, vp, tables, dl, 16, b.scale, ws, out=out, entry="pa_decode_split")
                ops.decode(q, kp, vp, tables, dl, 16, b.scale, ws, out=out, entry="pa_decode_reduce")
            else:
                ops.decode(q, kp, vp, tables, dl, 16, b.scale, ws, out=out)
        torch.cuda.synchronize()
        timings[entry] = (time.perf_counter() - t0) / 5 * 1e6
    print(f"[timing] one launch {timings['pa_decode']:.1f} us, split + reduce {timings['two']:.1f} us", flush=True)
    assert timings["pa_decode"] < 4 * timings["two"] + 200, "the merge of the long sequence's pieces dominates the launch"


@pytest.mark.parametrize("batch,long_len,short", [(200, 4000, 300), (128, 30000, 200), (160, 1500, 700)])
def test_sequences_of_many_pieces_are_merged_in_groups(batch, long_len, short):
    """A sequence cut into more than eight pieces is merged in two levels (groups of 8, 16 or 32 pieces, then the
    groups); here one sequence takes about 20, about 150 and about 5 pieces beside sequences of one or two."""
    announce(f"decode merge-in-split: groups of pieces, batch {batch}, one sequence of {long_len}")
    rng = np.random.default_rng(batch)
    lens = _ragged(rng, batch, short // 2, short)
    lens[batch // 3] = long_len
    b = Batch(lens, 32, 8, 128, "bf16", seed=batch)
    _three_ways(b, what=f"batch {batch} with one sequence of {long_len}")
    # (an fp8 pool of 8 kv heads is one plane: it takes the one-launch path from 64 sequences on)
    kv = "fp8" if _passes(batch, 32, 8, 128, torch.float8_e4m3fn) == 1 else "f16"
    b = Batch(lens, 32, 8, 128, kv, seed=batch + 1)
    _three_ways(b, extra_zero=[max(b.lens) - n for n in b.lens], what=f"{kv}, batch {batch}, extra zero keys")


def test_more_sequences_than_one_launch_takes():
    """Above 8192 sequences the call runs 8192 at a time on the stream."""
    announce("decode batch 8200 (two groups)")
    rng = np.random.default_rng(8)
    lens = _ragged(rng, 8200, 0, 40)
    b = Batch(lens, 4, 2, 32, "f32", seed=2)
    (kp, vp, _, _), _ = b.device_pools()
    q = b.q.to(DEV)
    got = ops.decode(q, kp, vp, tables_to_device(b.tables), torch.tensor(b.lens, dtype=torch.int32, device=DEV), 16,
                     b.scale, ops.decode_workspace(q, kp))
    want = po.paged_decode(b.q, b.k, b.v, b.tables, b.lens, 16, b.scale)
    assert_close(got, want, 1e-5, "batch 8200")


@pytest.mark.parametrize("kv,static", [("bf16", False), ("fp8", False), ("bf16", True)])
def test_append_and_decode_of_256_sequences_replayed_from_a_graph(kv, static):
    """One captured step (append, then decode) replayed with lengths, slots, queries and new rows rewritten in
    place; between the replays eager calls of other shapes use the same workspace (or the library's scratch).
    Every replay is checked against the checker; a replay finds the tickets as the previous launch left them."""
    announce(f"decode merge-in-split in a HIP graph {kv} static={static}")
    rng = np.random.default_rng(31)
    batch, hq, hkv, d, bs = 256, 32, 8, 128, 16
    room = 12  # blocks per sequence
    start = rng.integers(0, 150, batch)
    start[[3, 40]] = 0  # two sequences start empty (their first appended token is their first key)
    nb = batch * room + 8
    perm = rng.permutation(nb)
    tables = perm[: batch * room].reshape(batch, room).astype(np.int32)
    dtype = torch.bfloat16
    draw = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(dtype)
    k_ref, v_ref = draw(nb * bs, hkv, d), draw(nb * bs, hkv, d)
    fp8 = kv == "fp8"
    if fp8:
        kc, ksc = ops.quantize_kv_e4m3(k_ref.to(DEV), bs)
        vc, vsc = ops.quantize_kv_e4m3(v_ref.to(DEV), bs)
    else:
        kc, vc, ksc, vsc = k_ref.to(DEV), v_ref.to(DEV), None, None
    assert _passes(batch, hq, hkv, d, kc.dtype) == 1
    q = torch.zeros(batch, hq, d, dtype=dtype, device=DEV)
    k_new, v_new = torch.zeros(batch, hkv, d, dtype=dtype, device=DEV), torch.zeros(batch, hkv, d, dtype=dtype, device=DEV)
    lens = start.astype(np.int32).copy()
    lens_dev = torch.from_numpy(lens).to(DEV)
    slots_dev = torch.full((batch,), -1, dtype=torch.int64, device=DEV)  # the warm-up step appends nothing
    tables_dev = torch.from_numpy(tables).to(DEV)
    out = torch.empty_like(q)
    ws = ops.decode_workspace(q, kc)

    def step():
        if fp8:
            touched = torch.div(slots_dev, bs, rounding_mode="floor").to(torch.int32)
            ops.kv_append_e4m3(kc, vc, ksc, vsc, k_new, v_new, slots_dev, bs, touched)
        else:
            ops.kv_scatter(kc, vc, k_new, v_new, slots_dev)
        if static:
            ops.decode_static(q, kc, vc, tables_dev, lens_dev, bs, d ** -0.5, None, ksc, vsc, out=out)
        else:
            ops.decode(q, kc, vc, tables_dev, lens_dev, bs, d ** -0.5, ws, None, ksc, vsc, out=out)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # warm-up outside the capture (pa_decode_static asks for its scratch address here)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    other = Batch(_ragged(rng, 150, 1, 500), hq, hkv, d, "bf16", seed=77)  # eager calls between the replays
    (okp, ovp, _, _), _ = other.device_pools()
    oq, otab = other.q.to(DEV), tables_to_device(other.tables)
    olen = torch.tensor(other.lens, dtype=torch.int32, device=DEV)
    owant = po.paged_decode(other.q, other.k, other.v, other.tables, other.lens, bs, other.scale)
    for it in range(5):
        lens += 1  # every sequence appends one token, then attends it
        qh, kh, vh = draw(batch, hq, d), draw(batch, hkv, d), draw(batch, hkv, d)
        slots = tables[np.arange(batch), (lens - 1) // bs].astype(np.int64) * bs + (lens - 1) % bs
        q.copy_(qh.to(DEV)); k_new.copy_(kh.to(DEV)); v_new.copy_(vh.to(DEV))
        lens_dev.copy_(torch.from_numpy(lens).to(DEV)); slots_dev.copy_(torch.from_numpy(slots).to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        if fp8:
            kd = po.dequantize_kv_e4m3(kc.cpu().view(torch.uint8), ksc.cpu(), bs)
            vd = po.dequantize_kv_e4m3(vc.cpu().view(torch.uint8), vsc.cpu(), bs)
        else:
            k_ref[slots] = kh
            v_ref[slots] = vh
            assert torch.equal(kc.cpu(), k_ref)
            kd, vd = k_ref, v_ref
        want = po.paged_decode(qh, kd, vd, [t.tolist() for t in tables], lens.tolist(), bs, d ** -0.5)
        assert_close(out, want, 6e-2 if fp8 else 2e-2, f"replay {it}")
        # eager work in between: another batch (150 sequences: one launch as well) through the same workspace /
        # the same scratch, which moves every region of the layout but the tickets
        if static:
            eager = ops.decode_static(oq, okp, ovp, otab, olen, bs, other.scale)
        else:
            eager = ops.decode(oq, okp, ovp, otab, olen, bs, other.scale, ws)
        assert_close(eager, owant, 2e-2, f"eager call after replay {it}")
