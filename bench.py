#!/usr/bin/env python3
"""Benchmark of the paged decode-attention hot path on one MI355X.

One step = one ``pa_decode`` call over one batch of the synthetic workload,
inputs resident in HBM.  The headline workload is workload c4 (Llama-3-8B
shape, B=256, bf16 pool, lognormal context lengths, seed 1004).  Prints one
JSON line; with the default workload the line also carries short runs of the
other configurations (c2, c5 decode; c3 append + chunked prefill; the c3 shape at
head_dim 256 and 64; dense prefill of 64 x 512 and 4 x 8192 tokens; one chunk
behind 200 000 cached keys at head_dim 128 and 256) under ``secondary``.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-secondary]
                    [--workload c4|c2|c5|c1|c3|c3-d256|c3-d64|c3-d96|long-d128|long-d256|dense-64x512|dense-4x8192|engine]
    python bench.py --traffic-from-pmc NAME KERNEL FETCH.csv WRITE.csv   # refresh profiles/traffic.json
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, vendor figure
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak, vendor figure

# HBM traffic of one launch of each workload's dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# scaled by a device copy of known size in the same run: written by `--traffic-from-pmc` from the counter files,
# never typed in; a workload without an entry reports null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def calibration_copy(dev) -> None:
    """One device copy of 1 GiB (reads 1 GiB, writes 1 GiB): what `--traffic-from-pmc` scales the counters by."""
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def measured_traffic(name):
    try:
        with open(TRAFFIC_FILE) as f:
            entry = json.load(f).get(name)
    except (OSError, ValueError):
        return None
    return None if entry is None else entry["bytes"]


def traffic_from_pmc(name, kernel, fetch_csv, write_csv) -> int:
    """Average FETCH_SIZE / WRITE_SIZE (KiB per dispatch) of `kernel` in two rocprofv3 counter_collection CSVs,
    each scaled by what the same counter reads for the 1 GiB device copy of `--copy-calibration` in the same file;
    stores the sum as workload `name` in profiles/traffic.json."""
    import csv

    def one(path, counter, copied_kib):
        mine, copy = [], []
        with open(path) as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] != counter:
                    continue
                if kernel in r["Kernel_Name"]:
                    mine.append(float(r["Counter_Value"]))
                elif "copyBuffer" in r["Kernel_Name"]:
                    copy.append(float(r["Counter_Value"]))
        if not mine or not copy:
            raise SystemExit(f"{path}: no {counter} rows for {kernel!r} or for the calibration copy")
        # the calibration copy (1 GiB, in one dispatch or split in two) is the largest device copy of the run
        big = [c for c in copy if c >= 0.9 * max(copy)]
        factor = copied_kib / sum(big)
        return sum(mine) / len(mine) * factor * 1024.0, factor

    fetch, f_scale = one(fetch_csv, "FETCH_SIZE", 1024 * 1024)
    write, w_scale = one(write_csv, "WRITE_SIZE", 1024 * 1024)
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        table = {}
    table[name] = {"bytes": int(round(fetch + write)), "kernel": kernel, "fetch_bytes": int(round(fetch)),
                   "write_bytes": int(round(write)), "fetch_scale": round(f_scale, 4), "write_scale": round(w_scale, 4)}
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps({name: table[name]}))
    return 0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c4", choices=["c1", "c2", "c3", "c3-d256", "c3-d64", "c3-d96", "long-d128", "long-d256", "dense-64x512",
                                                         "dense-4x8192", "c4", "c5", "engine"])
    ap.add_argument("--preheat-s", type=float, default=0.5,
                    help="seconds of untimed steps before the warmup steps: an idle GPU sits at its lowest clocks "
                         "and takes a few hundred milliseconds of work to leave them")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="rough budget of the CPU baseline sample")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy, as the known-size kernel HBM counters are scaled by")
    ap.add_argument("--no-secondary", action="store_true",
                    help="with the default workload: leave out the short runs of c2, c5 and c3")
    ap.add_argument("--traffic-from-pmc", nargs=4, metavar=("NAME", "KERNEL", "FETCH_CSV", "WRITE_CSV"),
                    help="no benchmark: compute a workload's HBM traffic from two rocprofv3 counter files")
    return ap.parse_args()


def cpu_baseline(w, budget_s: float):
    """Time the vectorised CPU restatement (index gather + SDPA per sequence) on a bounded sample."""
    from oracle import paged_oracle as po

    threads = torch.get_num_threads()
    order = np.argsort(w.seq_lens)  # shortest first so the sample can be cut to the budget
    tables = [w.block_tables[i].tolist() for i in order]
    lens = w.seq_lens[order]
    q = w.q[torch.from_numpy(order)][:, None]
    k_pool, v_pool = w.k_pool, w.v_pool
    if w.kv_format == "fp8_e4m3":  # the CPU path of the fp8 workload is dequantise-then-attend
        kb, ks = po.quantize_kv_e4m3(k_pool, w.block_size)
        vb, vs = po.quantize_kv_e4m3(v_pool, w.block_size)
        k_pool = po.dequantize_kv_e4m3(kb, ks, w.block_size).to(w.dtype)
        v_pool = po.dequantize_kv_e4m3(vb, vs, w.block_size).to(w.dtype)
    po.decode_per_sequence(q[:2], k_pool, v_pool, tables[:2], lens[:2], w.block_size, w.scale)  # warm up
    done_tokens, done_seqs, at, t0 = 0, 0, 0, time.perf_counter()
    # walk the batch (again from the start once it is exhausted) until the budget is used
    while time.perf_counter() - t0 < budget_s:
        n = min(4, len(lens) - at)
        sl = slice(at, at + n)
        po.decode_per_sequence(q[sl], k_pool, v_pool, tables[sl], lens[sl], w.block_size, w.scale)
        done_seqs += n
        done_tokens += int(lens[sl].sum())
        at = (at + n) % len(lens)
    dt = time.perf_counter() - t0
    # the same bytes per key as the GPU figure counts: one per element of an fp8 pool (the CPU path itself reads
    # the dequantised 16-bit copy)
    kv_size = 1 if w.kv_format == "fp8_e4m3" else w.q.element_size()
    sample_bytes = done_tokens * w.num_kv_heads * w.head_dim * 2 * kv_size
    return {
        "value": sample_bytes / dt / 1e9,
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "tokens_per_s": done_seqs / dt,
        "sample": f"{done_seqs} sequence passes over the {len(lens)} sequences of {w.name}, shortest first, "
                  f"cycling ({done_tokens} keys), per-sequence index gather + torch SDPA on {threads} threads, "
                  f"{dt:.1f} s",
    }


def cpu_literal(w):
    """One pass of the literal restatement of the reference's decode (token-by-token gather loop into a
    zero-padded batch, repeat_interleave, unmasked SDPA) over the whole workload; only for the workloads small
    enough to run it as written (c1, c2)."""
    from oracle import paged_oracle as po

    tables = [t.tolist() for t in w.block_tables]
    t0 = time.perf_counter()
    po.decode_literal(w.q[:, None], w.k_pool, w.v_pool, tables, w.seq_lens, w.block_size, w.scale)
    dt = time.perf_counter() - t0
    padded = 2 * w.batch * int(w.seq_lens.max()) * w.num_q_heads * w.head_dim * w.q.element_size()
    return {"value": w.algorithmic_bytes() / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port", "seconds": dt, "tokens_per_s": w.batch / dt,
            "sample": f"the whole of {w.name} once: {2 * int(w.seq_lens.sum())} row copies issued from Python, "
                      f"{padded / 1e9:.2f} GB of padded and head-expanded K/V, one SDPA call"}


def preheat(fn, seconds):
    """Untimed calls of `fn` for about `seconds`, so that the timed region does not start on idle clocks."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def timed_ms(fn, steps):
    """Average milliseconds per call: HIP events on the launch stream around `steps` calls."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def timed_steps(fn, steps):
    """(mean, median) milliseconds per call over exactly `steps` calls: one HIP event on the launch stream before
    the first call and one behind every call; the mean is the whole bracket, the median is over the steps."""
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    marks[0].record()
    for i in range(steps):
        fn()
        marks[i + 1].record()
    torch.cuda.synchronize()
    each = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    return marks[0].elapsed_time(marks[steps]) / steps, each[steps // 2]


KERNEL_LAUNCHES = 50  # launches the dominant kernel's average duration is taken over


def bench_prefill_c3(args, dev) -> dict:
    """Workload c3: append 32 x 256 new K/V rows, then chunked causal prefill over 2048 shared prefix keys.

    One step = pa_kv_scatter + pa_prefill_paged.  The value is the step's attention FLOP rate; the roofline
    entry is the matrix-core prefill kernel alone; the append is reported beside it in GB/s.
    """
    from oracle import paged_oracle as po
    from research_amd import ops
    from research_amd.workloads import make_prefill_c3

    w = make_prefill_c3()
    S, C, P = w.num_seqs, w.chunk_len, w.prefix_len
    shape = (w.num_blocks * w.block_size, w.num_kv_heads, w.head_dim)
    kc = torch.zeros(shape, dtype=w.dtype, device=dev)
    vc = torch.zeros_like(kc)
    ops.kv_scatter(kc, vc, w.k_prefix.to(dev), w.v_prefix.to(dev), torch.from_numpy(w.prefix_slots()).to(dev))
    k_new = w.k_chunk.reshape(S * C, *shape[1:]).to(dev)
    v_new = w.v_chunk.reshape(S * C, *shape[1:]).to(dev)
    slots = torch.from_numpy(w.chunk_slots()).to(dev)
    q = w.q.reshape(S * C, w.num_q_heads, w.head_dim).to(dev)
    tables = torch.from_numpy(np.stack(w.block_tables).astype(np.int32)).to(dev)
    ctx = torch.full((S,), P + C, dtype=torch.int32, device=dev)
    ql = torch.full((S,), C, dtype=torch.int32, device=dev)
    qs = torch.arange(S, dtype=torch.int32, device=dev) * C
    out = torch.empty_like(q)

    def append():
        ops.kv_scatter(kc, vc, k_new, v_new, slots)

    def prefill():
        ops.prefill_paged(q, kc, vc, tables, ctx, ql, qs, C, w.block_size, w.scale, out=out)

    def step():
        append()
        prefill()

    if args.copy_calibration:
        calibration_copy(dev)
    preheat(step, args.preheat_s)
    for _ in range(args.warmup):
        step()
    ms_step_mean, ms_step = timed_steps(step, args.steps)
    ms_prefill = timed_ms(prefill, max(args.steps, KERNEL_LAUNCHES))
    ms_append = timed_ms(append, max(args.steps, KERNEL_LAUNCHES))
    # The same append with the rotary embedding of q and k fused in (the step a model runs right before this
    # path), beside the two-pass form: rotation into dense buffers, then the scatter.
    pos = (torch.arange(C, dtype=torch.int32, device=dev) + P).repeat(S)
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, w.head_dim, 2, device=dev).float() / w.head_dim))
    angles = torch.arange(P + C, device=dev).float()[:, None] * inv_freq[None, :]
    cos_t = torch.cat((angles, angles), dim=-1).cos().to(w.dtype)
    sin_t = torch.cat((angles, angles), dim=-1).sin().to(w.dtype)
    q_rot, k_rot = torch.empty_like(q), torch.empty_like(k_new)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)  # scratch pool: the timed pool keeps its unrotated rows

    def rope_fused():
        ops.rope_kv_append(q, k_new, v_new, cos_t, sin_t, kc2, vc2, slots, positions=pos, q_out=q_rot)

    def rope_two_pass():
        ops.rope_kv_append(q, k_new, v_new, cos_t, sin_t, None, None, None, positions=pos, q_out=q_rot, k_out=k_rot)
        ops.kv_scatter(kc2, vc2, k_rot, v_new, slots)

    preheat(rope_fused, 0.1)
    ms_rope = timed_ms(rope_fused, args.steps)
    ms_rope2 = timed_ms(rope_two_pass, args.steps)
    eb = q.element_size()
    rope_bytes = (2 * q.numel() + 4 * k_new.numel()) * eb + 2 * S * C * w.head_dim * eb + S * C * 12
    flops = w.attention_flops()
    achieved = flops / (ms_prefill * 1e-3) / 1e12
    result = {
        "metric": "prefill-attn TFLOP/s", "value": flops / (ms_step * 1e-3) / 1e12, "unit": "TFLOP/s",
        "tokens_per_s": S * C / (ms_step * 1e-3), "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "preheat_s": args.preheat_s, "ms_per_step": ms_step, "ms_per_step_mean": ms_step_mean, "step_statistic": "median of the timed steps",
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "c3 shared-prefix chunked prefill + KV append, 32 x (2048 + 256), bf16",
                   "num_seqs": S, "prefix_len": P, "chunk_len": C, "num_q_heads": w.num_q_heads,
                   "num_kv_heads": w.num_kv_heads, "head_dim": w.head_dim, "block_size": w.block_size,
                   "attention_flops": flops, "append_bytes": w.append_bytes(), "seed": 1003},
        "roofline": {"bound": "mfma", "kernel": "prefill_asm_kernel", "achieved": achieved,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": measured_traffic("c3"), "kernel_ms": ms_prefill,
                     "kernel_launches": max(args.steps, KERNEL_LAUNCHES)},
        "append": {"kernel": "kv_scatter_kernel", "kernel_ms": ms_append,
                   "achieved_gbps": w.append_bytes() / (ms_append * 1e-3) / 1e9, "peak_gbps": HBM_PEAK_GBPS},
        "rope_append": {"kernel": "rope_kv_append_kernel", "kernel_ms": ms_rope, "bytes": rope_bytes,
                        "achieved_gbps": rope_bytes / (ms_rope * 1e-3) / 1e9, "peak_gbps": HBM_PEAK_GBPS,
                        "two_pass_ms": ms_rope2},
    }
    if not args.no_cpu_baseline:
        threads = torch.get_num_threads()
        kcc, vcc = kc.cpu(), vc.cpu()
        n = 0  # sequence passes of the sample (cycling over the batch)
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < args.cpu_seconds:
            s = n % S
            blocks = np.asarray(w.block_tables[s])
            pos = np.arange(P + C)
            idx = torch.from_numpy(blocks[pos // w.block_size] * w.block_size + pos % w.block_size)
            k_full, v_full = kcc[idx][None], vcc[idx][None]
            q_full = torch.cat([torch.zeros(P, w.num_q_heads, w.head_dim, dtype=w.dtype), w.q[s]])[None]
            po.prefill_literal(q_full, k_full, v_full, w.scale)
            n += 1
        dt = time.perf_counter() - t0
        result["cpu_baseline"] = {
            "value": flops / S * n / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"{n} sequence passes over the {S} sequences (cycling): index gather of prefix+chunk, then the reference's full-sequence causal "
                      f"SDPA over {P + C} tokens (rows {P}..{P + C - 1} are the chunk), {threads} threads, {dt:.1f} s; "
                      "FLOPs counted for the chunk rows only",
        }
    return result


# the c3 shape at other head sizes: workload -> (query heads, kv heads, head_dim, seed, kernel)
PREFILL_HEAD_SHAPES = {"c3-d256": (16, 8, 256, 1006, "prefill_d256_kernel"),
                       "c3-d64": (32, 8, 64, 1007, "prefill_asm_kernel"),
                       # a head size between the compiled ones: the head_dim-128 kernel, rows of 96 in memory
                       "c3-d96": (32, 8, 96, 1011, "prefill_asm_kernel")}


def bench_prefill_head(args, dev, name) -> dict:
    """The c3 shape (32 x (2048 shared + 256 own) tokens, 16-token blocks, bf16) with 16 query / 8 kv heads of 256,
    or 32 query / 8 kv heads of 64 or 96: the chunked-prefill kernel for that head size alone, against the bf16
    matrix-core peak (head_dim 96 runs the head_dim-128 kernel; its FLOP count is that of 96)."""
    from research_amd import ops
    from research_amd.workloads import make_prefill_c3

    hq, hkv, head_dim, seed, kernel = PREFILL_HEAD_SHAPES[name]
    w = make_prefill_c3(num_q_heads=hq, num_kv_heads=hkv, head_dim=head_dim, seed=seed)
    S, C, P = w.num_seqs, w.chunk_len, w.prefix_len
    shape = (w.num_blocks * w.block_size, w.num_kv_heads, w.head_dim)
    kc = torch.zeros(shape, dtype=w.dtype, device=dev)
    vc = torch.zeros_like(kc)
    ops.kv_scatter(kc, vc, w.k_prefix.to(dev), w.v_prefix.to(dev), torch.from_numpy(w.prefix_slots()).to(dev))
    ops.kv_scatter(kc, vc, w.k_chunk.reshape(S * C, *shape[1:]).to(dev), w.v_chunk.reshape(S * C, *shape[1:]).to(dev),
                   torch.from_numpy(w.chunk_slots()).to(dev))
    q = w.q.reshape(S * C, w.num_q_heads, w.head_dim).to(dev)
    tables = torch.from_numpy(np.stack(w.block_tables).astype(np.int32)).to(dev)
    ctx = torch.full((S,), P + C, dtype=torch.int32, device=dev)
    ql = torch.full((S,), C, dtype=torch.int32, device=dev)
    qs = torch.arange(S, dtype=torch.int32, device=dev) * C
    out = torch.empty_like(q)

    def prefill():
        ops.prefill_paged(q, kc, vc, tables, ctx, ql, qs, C, w.block_size, w.scale, out=out)

    if args.copy_calibration:
        calibration_copy(dev)
    preheat(prefill, args.preheat_s)
    for _ in range(args.warmup):
        prefill()
    ms_step_mean, ms_step = timed_steps(prefill, args.steps)
    ms_kernel = timed_ms(prefill, max(args.steps, KERNEL_LAUNCHES))
    flops = w.attention_flops()
    achieved = flops / (ms_kernel * 1e-3) / 1e12
    return {
        "metric": "prefill-attn TFLOP/s", "value": flops / (ms_step * 1e-3) / 1e12, "unit": "TFLOP/s",
        "tokens_per_s": S * C / (ms_step * 1e-3), "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "preheat_s": args.preheat_s, "ms_per_step": ms_step, "ms_per_step_mean": ms_step_mean, "step_statistic": "median of the timed steps",
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"c3 shape at head_dim {head_dim}: chunked prefill, 32 x (2048 + 256), {hq} q / {hkv} kv heads, bf16",
                   "num_seqs": S, "prefix_len": P, "chunk_len": C, "num_q_heads": w.num_q_heads,
                   "num_kv_heads": w.num_kv_heads, "head_dim": w.head_dim, "block_size": w.block_size,
                   "attention_flops": flops, "seed": seed},
        "roofline": {"bound": "mfma", "kernel": kernel, "achieved": achieved,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": measured_traffic(name), "kernel_ms": ms_kernel,
                     "kernel_launches": max(args.steps, KERNEL_LAUNCHES)},
    }


# one long sequence: workload -> (query heads, kv heads, head_dim, seed, kernel)
PREFILL_LONG_SHAPES = {"long-d128": (8, 2, 128, 1008, "prefill_asm_kernel"),
                       "long-d256": (8, 2, 256, 1009, "prefill_d256_kernel")}


def bench_prefill_long(args, dev, name) -> dict:
    """A 2048-token chunk of ONE sequence behind 200 000 cached keys (16-token blocks in random pool order, bf16,
    8 query / 2 kv heads): more keys than the prefill kernels' LDS slot tables hold, so the instances that fill them
    again on the way run; few rows: 64 (head_dim 128) or 128 (256) workgroups for 256 CUs, so the call hands over a
    workspace and the head_dim 128 launch runs every workgroup's keys in pieces (kernel_ms then covers the piece
    kernel and the merge of the pieces)."""
    from research_amd import ops

    hq, hkv, head_dim, seed, kernel = PREFILL_LONG_SHAPES[name]
    P, C, bs = 200_000, 2048, 16
    nblk = -(-(P + C) // bs)
    gen = torch.Generator(device=dev).manual_seed(seed)
    kc = torch.randn(nblk * bs, hkv, head_dim, device=dev, dtype=torch.bfloat16, generator=gen)
    vc = torch.randn(nblk * bs, hkv, head_dim, device=dev, dtype=torch.bfloat16, generator=gen)
    q = torch.randn(C, hq, head_dim, device=dev, dtype=torch.bfloat16, generator=gen)
    tables = torch.randperm(nblk, device=dev, generator=gen).to(torch.int32).reshape(1, -1).contiguous()
    ctx = torch.tensor([P + C], dtype=torch.int32, device=dev)
    ql = torch.tensor([C], dtype=torch.int32, device=dev)
    qs = torch.zeros(1, dtype=torch.int32, device=dev)
    out = torch.empty_like(q)
    scale = head_dim ** -0.5

    # few rows: with a workspace the library cuts every workgroup's keys into pieces run side by side
    ws_bytes = ops.prefill_workspace_bytes(q, tables, C, bs, hkv)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    pieces = ws_bytes // (C * hq * (head_dim + 2) * 4)

    def prefill():
        ops.prefill_paged(q, kc, vc, tables, ctx, ql, qs, C, bs, scale, out=out, workspace=ws)

    if args.copy_calibration:
        calibration_copy(dev)
    preheat(prefill, args.preheat_s)
    for _ in range(args.warmup):
        prefill()
    ms_step_mean, ms_step = timed_steps(prefill, args.steps)
    ms_kernel = timed_ms(prefill, max(args.steps, KERNEL_LAUNCHES))
    flops = 4 * head_dim * hq * (C * P + C * (C + 1) // 2)  # two products, every visible (row, key) pair
    achieved = flops / (ms_kernel * 1e-3) / 1e12
    return {
        "metric": "prefill-attn TFLOP/s", "value": flops / (ms_step * 1e-3) / 1e12, "unit": "TFLOP/s",
        "tokens_per_s": C / (ms_step * 1e-3), "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "preheat_s": args.preheat_s, "ms_per_step": ms_step, "ms_per_step_mean": ms_step_mean, "step_statistic": "median of the timed steps",
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"one sequence, chunked prefill, 200000 + 2048, {hq} q / {hkv} kv heads of {head_dim}, bf16",
                   "num_seqs": 1, "prefix_len": P, "chunk_len": C, "num_q_heads": hq, "num_kv_heads": hkv,
                   "head_dim": head_dim, "block_size": bs, "attention_flops": flops, "seed": seed,
                   "key_pieces_per_workgroup": max(1, pieces), "workspace_bytes": ws_bytes},
        "roofline": {"bound": "mfma", "kernel": kernel, "achieved": achieved,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": measured_traffic(name), "kernel_ms": ms_kernel,
                     "kernel_launches": max(args.steps, KERNEL_LAUNCHES)},
    }


# dense causal prefill (no cached prefix): workload -> (sequences, tokens each, query heads, kv heads, head_dim, seed)
PREFILL_DENSE_SHAPES = {"dense-64x512": (64, 512, 32, 8, 128, 1010), "dense-4x8192": (4, 8192, 32, 8, 128, 1011)}


def bench_prefill_dense(args, dev, name) -> dict:
    """Dense causal prefill as ``_prefill_attention`` issues it: the step's own [B, T, Hkv, D] K/V handed to the
    paged kernel as a pool of B blocks of T tokens with the identity table.  64 prompts of 512 tokens are what an
    engine step of fresh prompts looks like: eight tiles of keys at most per workgroup, so the kernel's set-up and
    write-out weigh as much as its loop."""
    from research_amd import ops

    B, T, hq, hkv, head_dim, seed = PREFILL_DENSE_SHAPES[name]
    gen = torch.Generator(device=dev).manual_seed(seed)
    q = torch.randn(B * T, hq, head_dim, device=dev, dtype=torch.bfloat16, generator=gen)
    k = torch.randn(B * T, hkv, head_dim, device=dev, dtype=torch.bfloat16, generator=gen)
    v = torch.randn(B * T, hkv, head_dim, device=dev, dtype=torch.bfloat16, generator=gen)
    tables = torch.arange(B, dtype=torch.int32, device=dev).reshape(B, 1).contiguous()
    lens = torch.full((B,), T, dtype=torch.int32, device=dev)
    starts = torch.arange(B, dtype=torch.int32, device=dev) * T
    out = torch.empty_like(q)
    scale = head_dim ** -0.5

    def prefill():
        ops.prefill_paged(q, k, v, tables, lens, lens, starts, T, T, scale, out=out)

    if args.copy_calibration:
        calibration_copy(dev)
    preheat(prefill, args.preheat_s)
    for _ in range(args.warmup):
        prefill()
    ms_step_mean, ms_step = timed_steps(prefill, args.steps)
    ms_kernel = timed_ms(prefill, max(args.steps, KERNEL_LAUNCHES))
    flops = 4 * head_dim * hq * B * (T * (T + 1) // 2)  # two products, every visible (row, key) pair
    achieved = flops / (ms_kernel * 1e-3) / 1e12
    return {
        "metric": "prefill-attn TFLOP/s", "value": flops / (ms_step * 1e-3) / 1e12, "unit": "TFLOP/s",
        "tokens_per_s": B * T / (ms_step * 1e-3), "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "preheat_s": args.preheat_s, "ms_per_step": ms_step, "ms_per_step_mean": ms_step_mean,
        "step_statistic": "median of the timed steps", "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"dense causal prefill, {B} x {T} tokens, {hq} q / {hkv} kv heads of {head_dim}, bf16",
                   "num_seqs": B, "prefix_len": 0, "chunk_len": T, "num_q_heads": hq, "num_kv_heads": hkv,
                   "head_dim": head_dim, "attention_flops": flops, "seed": seed},
        "roofline": {"bound": "mfma", "kernel": "prefill_asm_kernel", "achieved": achieved,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": measured_traffic(name), "kernel_ms": ms_kernel,
                     "kernel_launches": max(args.steps, KERNEL_LAUNCHES)},
    }


def bench_engine(args, dev) -> int:
    """The engine loop on a Qwen2.5-0.5B-shaped model with random weights (24 layers, 14 query / 2 kv heads of
    64, vocabulary 151 936, bf16): 8 prompts of 512 tokens, 16 rollouts each, 64 new tokens per rollout at
    temperature 1.  One step = one whole ``generate`` call.  Timed for the paged path (radix allocator: the
    rollouts of a prompt share its prefix blocks) and, beside it, for the reference engine's own design, the
    cache-less loop that recomputes every sequence each step (engine.py:218-250), through the same model."""
    from research_amd.inference import (CacheConfig, EngineConfig, HipPagedAttentionBackend, InferenceEngine,
                                        ModelConfig, PagedLlama, SamplingParams)

    cfg = ModelConfig(vocab_size=151936, hidden_size=896, intermediate_size=4864, num_layers=24, num_heads=14,
                      num_kv_heads=2, head_dim=64, rope_theta=1e6, rms_norm_eps=1e-6, max_position_embeddings=2048,
                      tie_word_embeddings=True, attention_bias=True)
    n_prompts, n_rollouts, prompt_len, new_tokens = 8, 16, 512, 64
    g = torch.Generator().manual_seed(7)
    prompts = [torch.randint(0, cfg.vocab_size, (prompt_len,), generator=g).tolist() for _ in range(n_prompts)]
    batch = [p for p in prompts for _ in range(n_rollouts)]
    params = SamplingParams(temperature=1.0, max_tokens=new_tokens)
    backend = HipPagedAttentionBackend(CacheConfig(
        num_layers=cfg.num_layers, num_kv_heads=cfg.num_kv_heads, head_dim=cfg.head_dim, num_blocks=8192,
        block_size=16, device="cuda", dtype=torch.bfloat16))
    torch.manual_seed(0)
    model = PagedLlama(cfg, backend).to(torch.bfloat16).to(dev).eval()

    def run(cache_type, reps, use_graphs=False):
        engine = InferenceEngine(EngineConfig(model_path="", cache_type=cache_type, block_size=16,
                                              max_batch_size=len(batch), max_model_len=2048, num_kv_blocks=8192,
                                              use_graphs=use_graphs),
                                 model=model)
        times = []
        for _ in range(reps):
            engine.flush_cache()
            torch.manual_seed(1)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            samples = engine.generate(batch, params)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            assert len(samples) == len(batch) and all(len(s.completion_tokens) == new_tokens for s in samples)
        return times

    run("radix", max(1, args.warmup // 5))  # untimed
    eager = run("radix", max(1, args.steps // 10))
    paged = run("radix", max(1, args.steps // 10) + 1, use_graphs=True)[1:]  # the first call captures the graph
    recompute = run("none", 1)
    n_new = len(batch) * new_tokens
    best = min(paged)
    result = {
        "metric": "engine generated tokens/s", "value": n_new / best, "unit": "tokens/s", "n_gpus": 1,
        "steps": len(paged), "warmup": max(1, args.warmup // 5), "ms_per_step": 1e3 * best,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "engine: Qwen2.5-0.5B-shaped model, 8 prompts x 16 rollouts, 512 + 64 tokens",
                   "cache_type": "radix", "use_graphs": True, "block_size": 16, "sequences": len(batch),
                   "prompt_len": prompt_len, "new_tokens": new_tokens, "all_ms": [round(1e3 * t, 1) for t in paged]},
        "without_graphs": {"tokens_per_s": n_new / min(eager), "ms": 1e3 * min(eager)},
        "recompute_loop": {"tokens_per_s": n_new / recompute[0], "ms": 1e3 * recompute[0],
                           "note": "cache_type none: the reference engine's cache-less loop through the same model"},
        "speedup_over_recompute": recompute[0] / best,
    }
    print(json.dumps(result))
    return 0


def bench_decode(name, args, dev) -> dict:
    """One decode workload: the pa_decode step, its dominant kernel alone, the CPU restatement beside it."""
    from research_amd import _lib, ops
    from research_amd.workloads import make_decode

    t_gen = time.perf_counter()
    w = make_decode(name)
    t_gen = time.perf_counter() - t_gen

    q = w.q.to(dev)
    if w.kv_format == "fp8_e4m3":
        k_pool, k_scale = ops.quantize_kv_e4m3(w.k_pool.to(dev), w.block_size)
        v_pool, v_scale = ops.quantize_kv_e4m3(w.v_pool.to(dev), w.block_size)
    else:
        k_pool, v_pool, k_scale, v_scale = w.k_pool.to(dev), w.v_pool.to(dev), None, None
    tables = torch.from_numpy(w.padded_tables()).to(dev)
    lens = torch.from_numpy(w.seq_lens.astype(np.int32)).to(dev)
    ws = ops.decode_workspace(q, k_pool)
    out = torch.empty_like(q)
    # A workload whose K/V fit several times into HBM but not far beyond the 256 MB last-level cache is rotated
    # over 4 copies of its pools, so that no launch finds the previous launch's lines on chip.
    kv_bytes = 2 * k_pool.numel() * k_pool.element_size()
    n_pools = 4 if kv_bytes < (1 << 30) else 1
    pools = [(k_pool, v_pool)] + [(k_pool.clone(), v_pool.clone()) for _ in range(n_pools - 1)]
    turn = [0]
    # one launch (the split pass merges the pieces itself) or two (split pass, reduction pass)
    passes = int(_lib.load().pa_decode_passes(w.batch, w.num_q_heads, w.num_kv_heads, w.head_dim,
                                              ops.PA_DTYPE[k_pool.dtype]))

    def step(entry="pa_decode"):
        kp, vp = pools[turn[0] % n_pools]
        turn[0] += 1
        ops.decode(q, kp, vp, tables, lens, w.block_size, w.scale, ws, k_scale=k_scale, v_scale=v_scale,
                   out=out, entry=entry)

    if args.copy_calibration:
        calibration_copy(dev)
    preheat(step, args.preheat_s)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter()
    ms_step_mean, ms_step = timed_steps(step, args.steps)
    wall = time.perf_counter() - wall
    n_kernel = max(args.steps, KERNEL_LAUNCHES)
    # the dominant kernel alone: the split pass (with one launch per step it IS the step)
    ms_split = timed_ms(lambda: step("pa_decode" if passes == 1 else "pa_decode_split"), n_kernel)
    ms_reduce = None if passes == 1 else timed_ms(lambda: step("pa_decode_reduce"), n_kernel)

    host_path = None
    if w.kv_format != "fp8_e4m3" and not getattr(args, "secondary_run", False):
        # What a decode call costs through the backend class, host side included, by the form the context's
        # integer fields arrive in: the reference's tuples of tuples (converted block id by block id in Python),
        # padded int32 arrays, or device tensors (used in place).  A new context object per call, as a new step
        # brings; wall time of one call including the wait for the GPU, best of three.
        from research_amd.inference import CacheConfig, HipPagedAttentionBackend, InferenceContext

        be = HipPagedAttentionBackend(CacheConfig(num_layers=1, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim,
                                                  num_blocks=1, block_size=w.block_size, dtype=k_pool.dtype,
                                                  device=str(dev)))
        be.set_num_heads(w.num_q_heads)
        be.config = CacheConfig(num_layers=1, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim,
                                num_blocks=k_pool.shape[0] // w.block_size, block_size=w.block_size,
                                dtype=k_pool.dtype, device=str(dev))
        be.k_cache, be.v_cache = k_pool.unsqueeze(0), v_pool.unsqueeze(0)  # the workload's pools, not a copy
        q4 = q.unsqueeze(1)
        forms = {
            "tuples": lambda: (tuple(tuple(int(x) for x in t) for t in w.block_tables), tuple(int(n) for n in w.seq_lens)),
            "int32_arrays": lambda: (w.padded_tables(), w.seq_lens.astype(np.int32)),
            "device_tensors": lambda: (tables, lens),
        }
        host_path = {"unit": "ms per backend decode call, host and GPU", "kernel_ms": ms_step}
        for form, make in forms.items():
            best = None
            for _ in range(3):
                bt, sl = make()  # the caller's own bookkeeping, outside the timed call
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                be._decode_attention(q4, 0, InferenceContext(is_prefill=False, block_tables=bt, seq_lens=sl,
                                                             max_seq_len=int(w.seq_lens.max())))
                torch.cuda.synchronize()
                dt = (time.perf_counter() - t0) * 1e3
                best = dt if best is None else min(best, dt)
            host_path[form] = best
        del be

    gather = None
    if name in ("c1", "c2") and not getattr(args, "secondary_run", False):
        # the reference's own decode materialises this copy first (_gather_kv_from_cache): the block-table
        # gather into zero-padded [B, max_len, Hkv, D] tensors, bit-exact, bound by HBM
        max_len = int(w.seq_lens.max())
        gk = torch.empty((w.batch, max_len, w.num_kv_heads, w.head_dim), dtype=k_pool.dtype, device=dev)
        gv = torch.empty_like(gk)
        run_gather = lambda: ops.kv_gather(k_pool, v_pool, tables, lens, max_len, w.block_size, out=(gk, gv))
        for _ in range(3):
            run_gather()
        ms_gather = timed_ms(run_gather, args.steps)
        row = w.num_kv_heads * w.head_dim * k_pool.element_size()
        g_bytes = 2 * w.batch * max_len * row + 2 * w.total_tokens * row + 4 * int(sum(len(t) for t in w.block_tables)) + 4 * w.batch
        gather = {"kernel": "kv_gather_kernel", "kernel_ms": ms_gather, "bytes": g_bytes,
                  "achieved": g_bytes / (ms_gather * 1e-3) / 1e9, "unit": "GB/s",
                  "frac": g_bytes / (ms_gather * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                  "note": "written 2*B*max_len rows + read 2*sum(L) rows + tables"}
        del gk, gv

    alg_bytes = w.algorithmic_bytes()
    achieved = alg_bytes / (ms_split * 1e-3) / 1e9
    result = {
        "metric": "decode-attn HBM GB/s",
        "value": alg_bytes / (ms_step * 1e-3) / 1e9,
        "unit": "GB/s",
        "pct_of_hbm_peak": 100.0 * alg_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "tokens_per_s": w.batch / (ms_step * 1e-3),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "preheat_s": args.preheat_s,
        "ms_per_step": ms_step,
        "ms_per_step_mean": ms_step_mean,
        "step_statistic": "median of the timed steps",
        "value_at_mean": alg_bytes / (ms_step_mean * 1e-3) / 1e9,
        "wall_ms_per_step": wall * 1e3 / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("fp8-e4m3 KV, bf16 q" if w.kv_format == "fp8_e4m3" else
                  "bf16" if w.dtype == torch.bfloat16 else str(w.dtype).replace("torch.", "")),
        "data": "synthetic",
        "config": {
            "workload": {"c1": "c1 fp32 decode B=4", "c2": "c2 Qwen3-0.6B-shaped decode B=64 bf16",
                         "c4": "c4 Llama-3-8B-shaped decode B=256 bf16 paged KV",
                         "c5": "c5 long-context fp8-e4m3 KV decode B=8"}[name],
            "batch": w.batch, "num_q_heads": w.num_q_heads, "num_kv_heads": w.num_kv_heads,
            "head_dim": w.head_dim, "block_size": w.block_size, "total_keys": w.total_tokens,
            "max_len": int(w.seq_lens.max()), "kv_format": w.kv_format or str(w.dtype).replace("torch.", ""),
            "algorithmic_bytes": alg_bytes, "pool_copies_rotated": n_pools, "launches_per_step": passes,
            "seed": 1000 + int(name[1]), "generate_s": round(t_gen, 1),
        },
        "roofline": {
            "bound": "hbm", "kernel": "decode_split_kernel", "achieved": achieved, "peak": HBM_PEAK_GBPS,
            "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS, "traffic": measured_traffic(name),
            "kernel_ms": ms_split, "kernel_launches": n_kernel, "reduce_kernel_ms": ms_reduce,
        },
    }
    if gather is not None:
        result["gather"] = gather
    if host_path is not None:
        result["host_path"] = host_path
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, args.cpu_seconds)
        if name in ("c1", "c2") and args.cpu_seconds > 0 and not getattr(args, "secondary_run", False):
            result["cpu_baseline_literal"] = cpu_literal(w)
    return result


def secondary(args, dev) -> dict:
    """Short runs of the configurations that are not the headline: what the step costs, the dominant kernel
    against its roofline and a few seconds of the CPU restatement, per workload."""
    import copy

    short = copy.copy(args)
    short.steps, short.warmup, short.preheat_s = 30, 5, 0.3
    short.cpu_seconds = min(args.cpu_seconds, 4.0)
    short.copy_calibration = False
    short.secondary_run = True
    out = {}
    for name in ("c2", "c5", "c3", "c3-d256", "c3-d64", "c3-d96", "dense-64x512", "dense-4x8192", "long-d128", "long-d256"):
        r = (bench_prefill_c3(short, dev) if name == "c3" else bench_prefill_head(short, dev, name) if name in PREFILL_HEAD_SHAPES
             else bench_prefill_dense(short, dev, name) if name in PREFILL_DENSE_SHAPES
             else bench_prefill_long(short, dev, name) if name in PREFILL_LONG_SHAPES else bench_decode(name, short, dev))
        keep = ("metric", "value", "unit", "ms_per_step", "ms_per_step_mean", "steps", "warmup", "tokens_per_s",
                "dtype", "roofline", "cpu_baseline", "append", "pct_of_hbm_peak")
        entry = {k: r[k] for k in keep if k in r}
        entry["workload"] = r["config"]["workload"]
        out[name] = entry
        torch.cuda.empty_cache()
    return out


def main() -> int:
    args = parse_args()
    if args.traffic_from_pmc:
        return traffic_from_pmc(*args.traffic_from_pmc)
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path, run with --gpus 1", file=sys.stderr)
        return 2
    from research_amd import _lib

    _lib.load()  # no fallback: raises if the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "engine":
        return bench_engine(args, dev)
    if args.workload in PREFILL_HEAD_SHAPES:
        result = bench_prefill_head(args, dev, args.workload)
    elif args.workload in PREFILL_LONG_SHAPES:
        result = bench_prefill_long(args, dev, args.workload)
    elif args.workload in PREFILL_DENSE_SHAPES:
        result = bench_prefill_dense(args, dev, args.workload)
    else:
        result = bench_prefill_c3(args, dev) if args.workload == "c3" else bench_decode(args.workload, args, dev)
    if args.workload == "c4" and not args.no_secondary:
        torch.cuda.empty_cache()
        result["secondary"] = secondary(args, dev)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
