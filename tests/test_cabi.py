"""The C ABI without a GPU: the library loads, exports every symbol the header
declares, and rejects bad arguments with a status code and a message before it
touches any device (so none of these calls computes anything)."""

import ctypes
import os
import re

import pytest

from research_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "paged_attn.h")


def _declared_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(pa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared_functions()
    assert len(names) >= 10
    for name in names:
        assert hasattr(lib, name), f"{name} declared in paged_attn.h but not exported"


def test_binding_table_matches_header():
    assert sorted(_lib.SIGNATURES) == _declared_functions()


def test_version_and_dtype_sizes():
    lib = _lib.load()
    assert lib.pa_version() == 6
    assert [lib.pa_dtype_bytes(c) for c in (0, 1, 2, 3, 4, -1)] == [4, 2, 2, 1, 0, 0]


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(FileNotFoundError, match="no other implementation"):
        _lib.load(str(tmp_path / "libpaged_attn.so"))


FAKE = ctypes.c_void_p(0x1000)  # never dereferenced: every call below is rejected first


def _status(name, *args):
    lib = _lib.load()
    rc = getattr(lib, name)(*args)
    return rc, _lib.last_error()


def test_scatter_argument_errors():
    rc, msg = _status("pa_kv_scatter", FAKE, FAKE, FAKE, FAKE, FAKE, 4, 64, 8, 128, 3, None)
    assert rc == _lib.PA_ERR_INVALID_ARG and "elem_bytes" in msg
    rc, msg = _status("pa_kv_scatter", FAKE, FAKE, FAKE, FAKE, FAKE, -1, 64, 8, 128, 2, None)
    assert rc == _lib.PA_ERR_INVALID_ARG and "n_tokens" in msg
    rc, msg = _status("pa_kv_scatter", None, FAKE, FAKE, FAKE, FAKE, 4, 64, 8, 128, 2, None)
    assert rc == _lib.PA_ERR_INVALID_ARG and "NULL" in msg
    rc, msg = _status("pa_kv_scatter", FAKE, FAKE, FAKE, FAKE, FAKE, 4, 64, 1, 3, 1, None)
    assert rc == _lib.PA_ERR_INVALID_ARG and "multiple of 4" in msg
    # nothing to do is fine and needs no pointers
    assert _status("pa_kv_scatter", None, None, None, None, None, 0, 64, 8, 128, 2, None)[0] == _lib.PA_OK


def test_gather_argument_errors():
    rc, msg = _status("pa_kv_gather", FAKE, FAKE, FAKE, FAKE, FAKE, 4, FAKE, 2, 16, 8, 0, 8, 128, 2, None)
    assert rc == _lib.PA_ERR_INVALID_ARG and "block_size" in msg
    rc, msg = _status("pa_kv_gather", FAKE, FAKE, None, FAKE, FAKE, 4, FAKE, 2, 16, 8, 16, 8, 128, 2, None)
    assert rc == _lib.PA_ERR_INVALID_ARG and "NULL" in msg
    assert _status("pa_kv_gather", None, None, None, None, None, 0, None, 0, 0, 8, 16, 8, 128, 2, None)[0] == 0


def _decode_args(**kw):
    a = dict(q=FAKE, k=FAKE, v=FAKE, out=FAKE, bt=FAKE, bt_stride=4, lens=FAKE, ez=None, ks=None, vs=None,
             batch=2, hq=32, hkv=8, d=128, bs=16, nb=64, scale=0.088, window=0, qd=_lib.PA_BF16, kvd=_lib.PA_BF16,
             ws=FAKE, ws_bytes=1 << 30, stream=None)
    a.update(kw)
    return [a[k] for k in ("q", "k", "v", "out", "bt", "bt_stride", "lens", "ez", "ks", "vs", "batch", "hq", "hkv",
                           "d", "bs", "nb", "scale", "window", "qd", "kvd", "ws", "ws_bytes", "stream")]


def test_decode_argument_errors():
    rc, msg = _status("pa_decode", *_decode_args(hq=30))
    assert rc == _lib.PA_ERR_INVALID_ARG and "multiple of num_kv_heads" in msg
    rc, msg = _status("pa_decode", *_decode_args(bs=0))
    assert rc == _lib.PA_ERR_INVALID_ARG and "block_size" in msg
    for entry in ("pa_decode_split", "pa_decode_reduce"):
        rc, msg = _status(entry, *_decode_args(hq=30))
        assert rc == _lib.PA_ERR_INVALID_ARG
    rc, msg = _status("pa_decode", *_decode_args(d=100))  # (any multiple of 8 up to 256 has a kernel)
    assert rc == _lib.PA_ERR_UNSUPPORTED and "head_dim=100" in msg
    rc, msg = _status("pa_decode", *_decode_args(d=264))
    assert rc == _lib.PA_ERR_UNSUPPORTED
    rc, msg = _status("pa_decode", *_decode_args(qd=_lib.PA_F32))
    assert rc == _lib.PA_ERR_UNSUPPORTED  # q and pool types must match unless the pool is fp8
    rc, msg = _status("pa_decode", *_decode_args(kvd=_lib.PA_FP8_E4M3))
    assert rc == _lib.PA_ERR_INVALID_ARG and "k_scale" in msg
    rc, msg = _status("pa_decode", *_decode_args(ws_bytes=1024))
    assert rc == _lib.PA_ERR_WORKSPACE and "need" in msg
    rc, msg = _status("pa_decode", *_decode_args(ws=None))
    assert rc == _lib.PA_ERR_WORKSPACE
    # more than 8192 sequences are taken 8192 at a time through a workspace sized for 8192
    lib = _lib.load()
    assert (lib.pa_decode_workspace_bytes(10000, 32, 8, 128, _lib.PA_BF16)
            == lib.pa_decode_workspace_bytes(8192, 32, 8, 128, _lib.PA_BF16))
    rc, msg = _status("pa_decode", *_decode_args(batch=10000, ws_bytes=1024))
    assert rc == _lib.PA_ERR_WORKSPACE
    rc, msg = _status("pa_decode", *_decode_args(q=None))
    assert rc == _lib.PA_ERR_INVALID_ARG and "NULL" in msg
    assert _status("pa_decode", *_decode_args(batch=0, q=None, ws=None, ws_bytes=0))[0] == _lib.PA_OK


def test_decode_static_argument_errors():
    """The entry point without a workspace rejects bad arguments, and shapes whose partials exceed the library's
    fixed scratch array, before it touches a device."""
    static = lambda **kw: _decode_args(**kw)[:-3] + [None]
    rc, msg = _status("pa_decode_static", *static(hq=30))
    assert rc == _lib.PA_ERR_INVALID_ARG and "multiple of num_kv_heads" in msg
    rc, msg = _status("pa_decode_static", *static(d=100))
    assert rc == _lib.PA_ERR_UNSUPPORTED
    rc, msg = _status("pa_decode_static", *static(batch=8192))
    assert rc == _lib.PA_ERR_WORKSPACE and "scratch" in msg and "pa_decode_workspace_bytes" in msg
    assert _status("pa_decode_static", *static(batch=0, q=None))[0] == _lib.PA_OK


def test_decode_workspace_arithmetic():
    lib = _lib.load()
    small = lib.pa_decode_workspace_bytes(1, 1, 1, 32, _lib.PA_F32)
    c4 = lib.pa_decode_workspace_bytes(256, 32, 8, 128, _lib.PA_BF16)
    # (4096 + planes*batch) slots of hpw*NREP heads x (D+2) floats: shapes only, no lengths
    assert 0 < small < c4 and c4 >= (4096 + 2 * 256) * 16 * 130 * 4
    assert c4 % 256 == 0
    assert lib.pa_decode_workspace_bytes(256, 32, 8, 128, _lib.PA_FP8_E4M3) > 0
    assert lib.pa_decode_workspace_bytes(-1, 32, 8, 128, _lib.PA_BF16) == 0
    assert "pa_decode_workspace_bytes" in _lib.last_error()
    # head sizes between the compiled ones take the next larger kernel (and its workspace); odd ones have none
    assert (lib.pa_decode_workspace_bytes(4, 32, 8, 96, _lib.PA_BF16)
            == lib.pa_decode_workspace_bytes(4, 32, 8, 128, _lib.PA_BF16))
    assert lib.pa_decode_workspace_bytes(4, 32, 8, 100, _lib.PA_BF16) == 0
    assert lib.pa_decode_workspace_bytes(4, 30, 8, 128, _lib.PA_BF16) == 0


def test_prefill_and_quantize_argument_errors():
    args = [FAKE, FAKE, FAKE, FAKE, FAKE, 4, FAKE, FAKE, FAKE, None, 2, 16, 32, 8, 128, 16, 64, 0.088, 0,
            _lib.PA_FP8_E4M3, None]
    rc, msg = _status("pa_prefill_paged", *args)
    assert rc == _lib.PA_ERR_INVALID_ARG and "dtype" in msg
    args[-2] = _lib.PA_BF16
    args[14] = 84  # (not a multiple of 8: no kernel)
    rc, msg = _status("pa_prefill_paged", *args)
    assert rc == _lib.PA_ERR_UNSUPPORTED
    rc, msg = _status("pa_quantize_kv_e4m3", FAKE, FAKE, FAKE, 4, 16, 8, 128, _lib.PA_FP8_E4M3, None)
    assert rc == _lib.PA_ERR_INVALID_ARG and "src_dtype" in msg
    rc, msg = _status("pa_quantize_kv_e4m3", None, FAKE, FAKE, 4, 16, 8, 128, _lib.PA_F32, None)
    assert rc == _lib.PA_ERR_INVALID_ARG and "NULL" in msg
    append = [FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 5, FAKE, 2, None, None, 64, 16, 8, 128, _lib.PA_BF16, None]
    bad = list(append); bad[16] = _lib.PA_FP8_E4M3
    rc, msg = _status("pa_kv_append_e4m3", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "src_dtype" in msg
    bad = list(append); bad[13] = 1024
    rc, msg = _status("pa_kv_append_e4m3", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "block_size" in msg
    bad = list(append); bad[8] = None
    rc, msg = _status("pa_kv_append_e4m3", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "NULL" in msg
    bad = list(append); bad[10] = FAKE  # a row order without the block starts
    rc, msg = _status("pa_kv_append_e4m3", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "row_order" in msg
    bad = list(append); bad[7] = 0  # nothing to append: fine even with no device
    rc, msg = _status("pa_kv_append_e4m3", *bad)
    assert rc == _lib.PA_OK


def test_rope_argument_errors():
    rope = [FAKE, FAKE, FAKE, FAKE, None, FAKE, FAKE, FAKE, FAKE, None, 8, FAKE, 4, 64, 32, 8, 128, _lib.PA_BF16, None]
    bad = list(rope); bad[17] = _lib.PA_FP8_E4M3
    rc, msg = _status("pa_rope_kv_append", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "dtype" in msg
    bad = list(rope); bad[16] = 24  # half a head = 12 bf16 = 24 bytes
    rc, msg = _status("pa_rope_kv_append", *bad)
    assert rc == _lib.PA_ERR_UNSUPPORTED and "16 bytes" in msg
    bad = list(rope); bad[10] = 3  # 3 table rows for 4 tokens and no positions
    rc, msg = _status("pa_rope_kv_append", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "positions" in msg
    bad = list(rope); bad[11] = None  # no slots and no k_out
    rc, msg = _status("pa_rope_kv_append", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "nowhere" in msg
    bad = list(rope); bad[0] = None
    rc, msg = _status("pa_rope_kv_append", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "NULL" in msg
    bad = list(rope); bad[12] = 0
    assert _status("pa_rope_kv_append", *bad)[0] == _lib.PA_OK
    fp8 = [FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, None, 8, FAKE, 4, FAKE, 1, None, None, 64, 16, 32,
           8, 128, _lib.PA_BF16, None]
    bad = list(fp8); bad[19] = 1024
    rc, msg = _status("pa_rope_kv_append_e4m3", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "block_size" in msg
    bad = list(fp8); bad[11] = 2
    rc, msg = _status("pa_rope_kv_append_e4m3", *bad)
    assert rc == _lib.PA_ERR_INVALID_ARG and "positions" in msg
    bad = list(fp8); bad[13] = 0
    assert _status("pa_rope_kv_append_e4m3", *bad)[0] == _lib.PA_OK


def test_error_text_is_cleared_by_a_good_call():
    _status("pa_kv_scatter", FAKE, FAKE, FAKE, FAKE, FAKE, -1, 64, 8, 128, 2, None)
    assert _lib.last_error() != ""
    assert _status("pa_kv_scatter", None, None, None, None, None, 0, 64, 8, 128, 2, None)[0] == 0
    assert _lib.last_error() == ""


@pytest.mark.parametrize("script,generated", [("gen_prefill_loop.py", "prefill_mfma_loop.inc"),
                                              ("gen_prefill_loop_d256.py", "prefill_d256_loop.inc")])
def test_generated_prefill_loop_is_current(tmp_path, script, generated):
    """The committed assembly loops (head_dim 128: prefill_mfma_loop.inc; head_dim 256: prefill_d256_loop.inc) are
    what their generators write (the generators also check the instruction distances the hardware does not
    interlock, so a schedule that violates one cannot be committed)."""
    import os
    import subprocess
    import sys
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "research_amd", "csrc")
    out = tmp_path / "loop.inc"
    subprocess.run([sys.executable, os.path.join(csrc, script), str(out)], check=True, stdout=subprocess.DEVNULL)
    assert out.read_text() == open(os.path.join(csrc, generated)).read()
