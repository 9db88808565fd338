"""ctypes binding of ``libpaged_attn.so`` (signatures: ``include/paged_attn.h``).

The library is built in-tree next to this file by ``research_amd/build.py``.
There is no fallback: if it is missing, loading raises and every attention
call fails with that error.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from typing import Optional

LIB_NAME = "libpaged_attn.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

PA_OK = 0
PA_ERR_INVALID_ARG = -1
PA_ERR_UNSUPPORTED = -2
PA_ERR_WORKSPACE = -3
PA_ERR_HIP = -4

PA_F32, PA_BF16, PA_F16, PA_FP8_E4M3 = 0, 1, 2, 3

# name -> (restype, argtypes); mirrors include/paged_attn.h declaration by declaration
SIGNATURES = {
    "pa_version": (c_int, []),
    "pa_last_error": (c_char_p, []),
    "pa_dtype_bytes": (c_int, [c_int]),
    "pa_kv_scatter": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_void_p],
    ),
    "pa_kv_gather": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int, c_int64, c_int64, c_int,
         c_int, c_int, c_int, c_void_p],
    ),
    "pa_decode_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "pa_decode_passes": (c_int, [c_int, c_int, c_int, c_int, c_int]),
    "pa_decode": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int, c_int, c_int, c_int, c_int, c_int64, c_float, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "pa_decode_split": None,   # same signature as pa_decode, filled in below
    "pa_decode_reduce": None,
    "pa_prefill_paged": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
         c_int, c_int, c_int, c_int, c_int, c_int64, c_float, c_int, c_int, c_void_p],
    ),
    "pa_attend_masked": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
         c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int64, c_float, c_int, c_int, c_void_p,
         c_void_p, c_void_p],
    ),
    "pa_quantize_kv_e4m3": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "pa_kv_append_e4m3": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int, c_void_p,
         c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "pa_dequantize_blocks_e4m3": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "pa_rope_kv_append": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
         c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "pa_rope_kv_append_e4m3": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_void_p, c_int64, c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int,
         c_void_p],
    ),
}
SIGNATURES["pa_decode_split"] = SIGNATURES["pa_decode_reduce"] = SIGNATURES["pa_decode"]
SIGNATURES["pa_prefill_paged_rowwise"] = SIGNATURES["pa_prefill_paged"]
# pa_prefill_paged + total_q, workspace, workspace_bytes
SIGNATURES["pa_prefill_paged_ws"] = (c_int, SIGNATURES["pa_prefill_paged"][1] + [c_int64, c_void_p, c_size_t])
SIGNATURES["pa_prefill_workspace_bytes"] = (
    c_size_t, [c_int, c_int, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_int])
# pa_decode without the workspace pointer and size
SIGNATURES["pa_decode_static"] = (c_int, SIGNATURES["pa_decode"][1][:-3] + [c_void_p])


class PagedAttnError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, fn: str, status: int, message: str) -> None:
        super().__init__(f"{fn} failed with status {status}: {message}")
        self.fn, self.status, self.message = fn, status, message


_lib: Optional[ctypes.CDLL] = None


def load(path: Optional[str] = None) -> ctypes.CDLL:
    """Load the shared library once and attach the declared signatures."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    target = path or LIB_PATH
    if not os.path.exists(target):
        raise FileNotFoundError(
            f"{target} is missing: build it with `python -m research_amd.build` "
            "(hipcc --offload-arch=gfx950); this backend has no other implementation"
        )
    # The library needs libamdhip64.so.7.  PyTorch-ROCm ships its own copy under
    # that soname; importing torch first makes the loader bind this library to
    # the runtime torch already uses.  Loaded the other way round the process
    # ends up with two HIP runtimes and launches fail with "no ROCm-capable
    # device" on pointers that belong to the other one.
    import torch  # noqa: F401

    lib = ctypes.CDLL(target)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError names the missing symbol
        fn.restype, fn.argtypes = restype, argtypes
    if path is None:
        _lib = lib
    return lib


def last_error() -> str:
    return load().pa_last_error().decode("utf-8", "replace")


def check(fn: str, status: int) -> None:
    if status != PA_OK:
        raise PagedAttnError(fn, status, last_error())
