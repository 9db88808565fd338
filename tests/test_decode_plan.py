"""The split pass's bookkeeping without a GPU: ``research_amd/csrc/decode_plan.h`` (the header the kernels and the
host entry point use for the partition, the partial slots and the workspace layout) is compiled with g++ into a
replay of both passes (``tests/host/decode_plan_replay.cpp``) and run over ragged batches.  For every batch: each
(plane, sequence, block) is attended exactly once and by the workgroup ``owner_of`` names, every partial slot is
unique and inside the workspace, every piece the reduction pass (or the in-split merge's ticket count) expects was
written, and the workgroup's LDS fits."""

import ctypes
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "host", "decode_plan_replay.cpp")

SHAPES = [  # (Hq, Hkv, D, bytes per pool element)
    (32, 8, 128, 2), (16, 8, 128, 2), (8, 2, 64, 4), (32, 8, 128, 1), (14, 2, 64, 2), (4, 4, 32, 4), (16, 8, 256, 2),
    (64, 1, 128, 2), (8, 8, 128, 2), (96, 8, 128, 2), (7, 7, 32, 1),
]


@pytest.fixture(scope="module")
def replay(tmp_path_factory):
    lib = str(tmp_path_factory.mktemp("plan") / "libplan_replay.so")
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-o", lib, SRC], check=True)
    fn = ctypes.CDLL(lib).pa_plan_replay
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 9 + [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int]

    def run(lens, shape, block_size=16, window=0, grid=512, grid_cap=4096):
        lens = np.ascontiguousarray(lens, dtype=np.int32)
        stats = np.zeros(8, dtype=np.int64)
        err = ctypes.create_string_buffer(256)
        rc = fn(lens.ctypes.data, len(lens), *shape, block_size, window, grid, grid_cap, stats.ctypes.data, err, 256)
        assert rc == 0, f"{err.value.decode()} (B={len(lens)}, shape={shape}, bs={block_size}, window={window}, grid={grid})"
        return dict(zip(("units", "workgroups", "pieces", "in_place", "max_slot", "slot_cap", "max_pieces", "ws_bytes"),
                        stats.tolist()))
    return run


def test_baseline_configurations(replay):
    rng = np.random.default_rng(1004)
    c4 = np.clip(np.rint(np.exp(rng.normal(np.log(2048.0), 1.0, 256))), 64, 32768)
    s = replay(c4, (32, 8, 128, 2))
    assert s["workgroups"] == 512 and s["units"] == 2 * int(np.ceil(c4 / 16).sum())
    assert s["max_slot"] < 512 + 2 * 256 - 1          # the tight bound the library's own scratch is laid out for
    replay(c4, (32, 8, 128, 2), grid_cap=512)         # the layout pa_decode_static uses
    c5 = np.random.default_rng(1005).integers(65536, 131073, 8)
    s = replay(c5, (32, 8, 128, 1))
    assert s["in_place"] == 0 and s["max_pieces"] >= 512 // 8
    replay(np.random.default_rng(1002).integers(512, 4097, 64), (16, 8, 128, 2))
    replay([232, 157, 210, 5], (8, 2, 64, 4))


@pytest.mark.parametrize("seed", range(6))
def test_ragged_batches(replay, seed):
    rng = np.random.default_rng(seed)
    for _ in range(40):
        batch = int(rng.choice([1, 2, 3, 7, 33, 64, 256, 1000]))
        kind = rng.integers(0, 4)
        if kind == 0:
            lens = rng.integers(0, 40, batch)                        # many empty and one-block sequences
        elif kind == 1:
            lens = np.clip(np.rint(np.exp(rng.normal(6.0, 1.5, batch))), 0, 200000)
        elif kind == 2:
            lens = np.full(batch, int(rng.integers(1, 5000)))
        else:
            lens = rng.integers(0, 3000, batch) * (rng.random(batch) < 0.5)
        shape = SHAPES[int(rng.integers(len(SHAPES)))]
        grid = int(rng.choice([1, 2, 3, 17, 64, 512, 608, 4096]))
        window = int(rng.choice([0, 0, 1, 17, 512, 100000]))
        bs = int(rng.choice([16, 16, 1, 8, 64, 256]))
        s = replay(lens, shape, block_size=bs, window=window, grid=grid, grid_cap=max(grid, 4096) if rng.random() < 0.5 else grid)
        assert s["max_slot"] < s["slot_cap"]
        assert s["pieces"] + s["in_place"] >= (1 if s["units"] else 0)


def test_extremes(replay):
    replay([0], (32, 8, 128, 2))
    replay([1], (32, 8, 128, 2), grid=4096)
    replay(np.zeros(8192, dtype=np.int32), (32, 8, 128, 2))
    lens = np.full(8192, 17)
    s = replay(lens, (32, 8, 128, 2), grid=4096)
    assert s["workgroups"] == 4096 and s["max_slot"] < s["slot_cap"]
    s = replay(lens, (32, 8, 128, 2), grid=512, grid_cap=512)
    assert s["max_slot"] < s["slot_cap"]
    replay([131072] * 3, (32, 8, 128, 1), grid=4096)
    replay([1000000], (8, 8, 128, 2), grid=512, window=4096)
    one_long = np.concatenate([np.full(300, 5), [200000]])
    s = replay(one_long, (96, 8, 128, 2), grid=512)   # 12 query heads per kv head: two rep groups
    assert s["max_pieces"] > 100


def test_replay_notices_a_workspace_that_is_too_small(replay):
    """The checker is not vacuous: with fewer slots than the bound, a slot falls outside and the replay says so."""
    c5 = np.random.default_rng(1005).integers(65536, 131073, 8)
    with pytest.raises(AssertionError, match="outside the workspace"):
        replay(c5, (32, 8, 128, 1), grid=512, grid_cap=8)


def test_merge_in_split_rule_and_layout_match_the_library():
    """The library's workspace size is the plan's layout for the 4096-workgroup bound (same header)."""
    from research_amd import _lib

    lib = _lib.load()
    want = lib.pa_decode_workspace_bytes(256, 32, 8, 128, _lib.PA_BF16)
    slots = 4096 + 2 * 256
    align = lambda x: -(-x // 256) * 256
    tickets = 640 * 1024  # the fixed region at the start (PA_DECODE_TICKET_BYTES)
    assert want == tickets + align(257 * 4) + align(slots * 16 * 2 * 4) + align(slots * 16 * 128 * 4)
