#!/usr/bin/env python3
"""Writes tests/golden/allocator_traces.json: random operation traces of the
reference's block allocator and everything observable after each operation.

Runs in the build container only (the reference tree is not present anywhere
else).  It loads the single reference file cache/paged.py by path - that file
imports numpy and xxhash only - and never imports the reference package.  The
allocator is host-side integer bookkeeping whose long-run behaviour (freed
block revival wiping its record, the never-pruned hash map, growth only after
hash-complete blocks) no closed form pins; the hand-traced scenarios in
tests/test_host_allocator.py cover each quirk once, these traces cover their
interleavings.

    python tests/golden/make_allocator_traces.py
"""

import importlib.util
import json
import os
import random

REF = "/root/reference/rollouts/rollouts/inference/cache/paged.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "allocator_traces.json")


def load_reference_allocator():
    spec = importlib.util.spec_from_file_location("_ref_paged", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.PagedKVCache


def observe(cache, seq_ids):
    return {
        "free": list(cache.free_block_ids),
        "used": sorted(cache.used_block_ids),
        "refs": [b.ref_count for b in cache.blocks],
        "hashed": [b.hash != -1 for b in cache.blocks],
        "tables": {str(s): list(cache.get_block_ids(s)) for s in seq_ids},
        "cached": {str(s): cache.get_cached_tokens(s) for s in seq_ids},
        "map_size": len(cache.hash_to_block_id),
    }


def make_trace(PagedKVCache, seed, num_blocks, block_size, steps):
    rng = random.Random(seed)
    cache = PagedKVCache(num_blocks=num_blocks, block_size=block_size)
    prompts = [[rng.randrange(4) for _ in range(block_size * 3)] for _ in range(3)]  # few prefixes -> many hits
    live, next_id, ops = [], 0, []
    for _ in range(steps):
        kind = rng.choice(["alloc", "alloc", "free", "append", "append"])
        op = {"op": kind}
        try:
            if kind == "alloc":
                base = rng.choice(prompts)
                n = rng.randrange(1, len(base) + block_size)
                toks = (base + [rng.randrange(4) for _ in range(block_size)])[:n]
                if rng.random() < 0.3:
                    toks[rng.randrange(len(toks))] = 9
                op.update(seq=next_id, tokens=toks)
                if cache.can_allocate(len(toks)):
                    op["result"] = list(cache.allocate(next_id, toks))
                    live.append(next_id)
                else:
                    op["result"] = "cannot_allocate"
                next_id += 1
            elif kind == "free":
                if live:
                    s = live.pop(rng.randrange(len(live)))
                    op.update(seq=s)
                    cache.deallocate(s)
                else:
                    op.update(seq=12345)
                    cache.deallocate(12345)  # unknown id: no-op
                op["result"] = None
            else:
                if not live:
                    continue
                s = rng.choice(live)
                op.update(seq=s, token=rng.randrange(4))
                op["result"] = cache.append_token(s, op["token"])
        except Exception as e:  # recorded, the twin must raise the same type
            op["result"] = {"raises": type(e).__name__}
        op["after"] = observe(cache, live)
        op["num_free"] = cache.num_free_blocks()
        ops.append(op)
    return {"seed": seed, "num_blocks": num_blocks, "block_size": block_size, "ops": ops}


def main():
    PagedKVCache = load_reference_allocator()
    traces = [make_trace(PagedKVCache, seed, nb, bs, 60) for seed, nb, bs in
              [(1, 8, 2), (2, 12, 4), (3, 6, 2), (4, 24, 4), (5, 10, 3), (6, 16, 2)]]
    with open(OUT, "w") as f:
        json.dump(traces, f, separators=(",", ":"))
    print(f"wrote {OUT}: {sum(len(t['ops']) for t in traces)} operations")


if __name__ == "__main__":
    main()
