"""Replays operation traces recorded from the reference allocator
(tests/golden/allocator_traces.json, written by tests/golden/make_allocator_traces.py
from rollouts/rollouts/inference/cache/paged.py) against this package's twin."""

import json
import os

import pytest

from research_amd.inference import PagedKVCache

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "allocator_traces.json")


def _observe(cache, seq_ids):
    return {
        "free": list(cache.free_block_ids),
        "used": sorted(cache.used_block_ids),
        "refs": [b.ref_count for b in cache.blocks],
        "hashed": [b.hash != -1 for b in cache.blocks],
        "tables": {str(s): list(cache.get_block_ids(s)) for s in seq_ids},
        "cached": {str(s): cache.get_cached_tokens(s) for s in seq_ids},
        "map_size": len(cache.hash_to_block_id),
    }


with open(FIXTURE) as _f:
    TRACES = json.load(_f)


@pytest.mark.parametrize("trace", TRACES, ids=[f"seed{t['seed']}" for t in TRACES])
def test_allocator_replays_reference_trace(trace):
    cache = PagedKVCache(num_blocks=trace["num_blocks"], block_size=trace["block_size"])
    live = []
    assert len(trace["ops"]) > 40
    for n, op in enumerate(trace["ops"]):
        where = f"seed {trace['seed']} op {n} {op['op']}"
        expect = op["result"]
        try:
            if op["op"] == "alloc":
                if cache.can_allocate(len(op["tokens"])):
                    got = list(cache.allocate(op["seq"], op["tokens"]))
                    live.append(op["seq"])
                else:
                    got = "cannot_allocate"
            elif op["op"] == "free":
                cache.deallocate(op["seq"])
                if op["seq"] in live:
                    live.remove(op["seq"])
                got = None
            else:
                got = cache.append_token(op["seq"], op["token"])
        except Exception as e:
            got = {"raises": type(e).__name__}
        assert got == expect, where
        assert cache.num_free_blocks() == op["num_free"], where
        assert _observe(cache, live) == op["after"], where


def test_traces_exercise_the_quirks():
    """The fixture is only worth something if hits, revivals and appends all occur in it."""
    ops = [op for t in TRACES for op in t["ops"]]
    assert any(op["op"] == "alloc" and isinstance(op["result"], list) and
               op["after"]["cached"].get(str(op["seq"]), 0) > 0 for op in ops)  # prefix hits
    assert any(op["op"] == "append" and isinstance(op["result"], int) for op in ops)  # growth
    assert any(op["op"] == "append" and op["result"] is None for op in ops)  # no growth
    assert any(op["result"] == "cannot_allocate" for op in ops)
