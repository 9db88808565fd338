"""The bookkeeping of the matrix-core prefill launches without a GPU: ``research_amd/csrc/prefill_plan.h`` (the
header the host entry points and the kernels share) compiled with g++ into ``tests/host/prefill_plan_replay.cpp``.
The pieces a workgroup's tiles are cut into cover the tiles once; the groups that the workgroups of one (sequence,
kv head) run in turn cover the groups once and stay within what the launch was sized for; the split rule picks the
cheapest admissible split of its own cost model; the workspace size is the layout the kernels index."""

import ctypes
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "host", "prefill_plan_replay.cpp")


@pytest.fixture(scope="module")
def plan(tmp_path_factory):
    lib = str(tmp_path_factory.mktemp("pfplan") / "libprefill_plan_replay.so")
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-o", lib, SRC], check=True)
    dll = ctypes.CDLL(lib)
    dll.pa_plan_pieces.argtypes = [ctypes.c_int] * 3 + [ctypes.c_char_p, ctypes.c_int]
    dll.pa_plan_groups.argtypes = [ctypes.c_int] * 3 + [ctypes.POINTER(ctypes.c_int), ctypes.c_char_p, ctypes.c_int]
    dll.pa_plan_splits.argtypes = [ctypes.c_longlong, ctypes.c_int, ctypes.c_longlong, ctypes.c_int]
    dll.pa_plan_cost.argtypes = [ctypes.c_longlong, ctypes.c_int, ctypes.c_longlong, ctypes.c_int]
    dll.pa_plan_cost.restype = ctypes.c_longlong
    dll.pa_plan_ws_bytes.argtypes = [ctypes.c_longlong, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    dll.pa_plan_ws_bytes.restype = ctypes.c_ulonglong
    dll.pa_plan_groups_per_workgroup.argtypes = [ctypes.c_int, ctypes.c_longlong, ctypes.c_int, ctypes.c_int]
    return dll


def _ok(rc, err):
    assert rc == 0, err.value.decode()


def test_pieces_cover_the_tiles_once(plan):
    err = ctypes.create_string_buffer(256)
    rng = np.random.default_rng(0)
    for n_all in list(range(0, 40)) + rng.integers(40, 6000, 200).tolist():
        for n_splits in range(1, 9):
            _ok(plan.pa_plan_pieces(int(rng.integers(0, 3000)), int(n_all), n_splits, err, 256), err)


def test_groups_of_a_sequence_are_each_run_once(plan):
    """As the host sizes the launch: gpw groups per workgroup, ceil(groups / gpw) workgroups along y."""
    err = ctypes.create_string_buffer(256)
    most = ctypes.c_int(0)
    for groups in range(1, 130):
        for gpw in range(1, 9):
            n_chunks = -(-groups // gpw)
            # a shorter sequence of the same launch has fewer groups than the launch was sized for
            for group_end in {groups, max(1, groups // 2), max(1, groups - 1), 1}:
                _ok(plan.pa_plan_groups(group_end, n_chunks, gpw, ctypes.byref(most), err, 256), err)
            _ok(plan.pa_plan_groups(groups, n_chunks, gpw, ctypes.byref(most), err, 256), err)
            assert most.value == -(-groups // n_chunks)


def test_zigzag_order_balances_causal_work(plan):
    """Group g of a dense causal prompt runs g + 1 tiles: with the groups dealt from the front in even rounds and
    from the back in odd ones the workgroups' tile counts differ by less than one round's spread."""
    groups, gpw = 64, 8
    n_chunks = groups // gpw
    totals = []
    for chunk in range(n_chunks):
        mine = [i * n_chunks + (n_chunks - 1 - chunk if i & 1 else chunk) for i in range(gpw)]
        totals.append(sum(g + 1 for g in mine))
    assert max(totals) - min(totals) == 0
    straight = [sum(i * n_chunks + chunk + 1 for i in range(gpw)) for chunk in range(n_chunks)]
    assert max(straight) - min(straight) == gpw * (n_chunks - 1)


@pytest.mark.parametrize("cus", [256, 304, 64])
def test_split_rule_is_the_cheapest_admissible_split(plan, cus):
    rng = np.random.default_rng(cus)
    for _ in range(400):
        workgroups = int(rng.integers(1, 4 * cus))
        max_keys = int(rng.integers(64, 400000))
        s = plan.pa_plan_splits(workgroups, cus, max_keys, 64)
        tiles = max_keys // 64
        assert 1 <= s <= 8
        if s > 1:
            assert tiles // s >= 24  # a piece keeps enough tiles to pay for its set-up
        cost = lambda k: plan.pa_plan_cost(workgroups, cus, tiles, k)
        admissible = [k for k in range(1, 9) if k == 1 or tiles // k >= 24]
        # (the rule stops at the first split that is too fine, so the admissible ones are 1 .. some k)
        assert admissible == list(range(1, len(admissible) + 1))
        assert cost(s) == min(cost(k) for k in admissible)
        assert all(cost(k) > cost(s) for k in admissible if k < s)  # the smaller on ties
    # launches that fill the device several times over stay whole; the long-context shapes of bench.py split
    assert plan.pa_plan_splits(64 * cus, cus, 1 << 20, 64) == 1
    assert plan.pa_plan_splits(64, 256, 202048 + 256, 64) == 4      # long-d128: 64 workgroups on 256 compute units
    assert plan.pa_plan_splits(128, 256, 202048 + 256, 64) == 2     # long-d256
    assert plan.pa_plan_splits(512, 256, 2304, 64) == 1             # c3


def test_workspace_size_is_the_layout_the_kernels_index(plan):
    # part_o float[row][head][piece][D] + part_ml float[row][head][piece][2]
    for total_q, hq, d, s in [(2048, 8, 128, 4), (150, 8, 256, 2), (7, 3, 32, 8)]:
        assert plan.pa_plan_ws_bytes(total_q, hq, d, s) == total_q * hq * s * (d + 2) * 4
    assert plan.pa_plan_ws_bytes(2048, 8, 128, 1) == 0 and plan.pa_plan_ws_bytes(2048, 8, 128, 0) == 0


def test_groups_per_workgroup_leaves_a_workgroup_per_compute_unit(plan):
    rng = np.random.default_rng(3)
    for _ in range(500):
        hkv, groups, batch, cus = int(rng.integers(1, 17)), int(rng.integers(1, 200)), int(rng.integers(1, 300)), 256
        g = plan.pa_plan_groups_per_workgroup(hkv, groups, batch, cus)
        assert 1 <= g <= min(8, groups)
        fills = lambda k: hkv * -(-groups // k) * batch >= cus
        assert g == 1 or fills(g)
        assert all(not fills(k) for k in range(g + 1, min(8, groups) + 1))
    assert plan.pa_plan_groups_per_workgroup(8, 8, 64, 256) == 8    # dense 64 x 512
    assert plan.pa_plan_groups_per_workgroup(8, 4, 32, 256) == 4    # c3: all 4 groups of a (sequence, kv head)
    assert plan.pa_plan_groups_per_workgroup(2, 8, 1, 256) == 1     # one long chunk: nothing to spare
