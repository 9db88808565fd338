"""Helpers shared by the GPU parity tests: move a synthetic workload to the
device and run the C-ABI entry points on it (through research_amd.ops)."""

import numpy as np
import torch

from research_amd import ops

DEV = "cuda:0"


def announce(msg):
    """Name the case before its first kernel launch, flushed, so a fault can be attributed."""
    print(f"[gpu-case] {msg}", flush=True)


def tables_to_device(tables, width=None):
    w = max(max((len(t) for t in tables), default=1), 1) if width is None else width
    out = np.full((len(tables), w), -1, dtype=np.int32)
    for i, t in enumerate(tables):
        out[i, : len(t)] = np.asarray(t, dtype=np.int64)
    return torch.from_numpy(out).to(DEV)


def run_decode(q, k_pool, v_pool, tables, seq_lens, block_size, scale, extra_zero=None, k_scale=None, v_scale=None,
               wgs_per_call=None):
    """q [B,Hq,D] and pools already on the device; tables/seq_lens host lists.  Returns a device tensor."""
    lens = np.asarray(seq_lens, dtype=np.int32)
    ws = ops.decode_workspace(q, k_pool)
    ez = None if extra_zero is None else torch.from_numpy(np.asarray(extra_zero, dtype=np.int32)).to(DEV)
    return ops.decode(q, k_pool, v_pool, tables_to_device(tables), torch.from_numpy(lens).to(DEV), block_size, scale,
                      ws, ez, k_scale, v_scale)


def assert_close(got, want, tol, what=""):
    """|got - want| <= tol * (1 + |want|): the absolute/relative bar used for attention outputs."""
    got = got.detach().to(torch.float64).cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got)
    want = want.detach().to(torch.float64).cpu().numpy() if isinstance(want, torch.Tensor) else np.asarray(want)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - want) / (1.0 + np.abs(want))
    assert err.max() <= tol, f"{what}: max err {err.max():.3e} > {tol:.1e} at {np.unravel_index(err.argmax(), err.shape)}"
