"""Host-side behaviour of the backend class that needs no GPU: construction,
attribute surface and the error conventions of the reference
(rollouts/rollouts/inference/attention/flex_backend.py)."""

import pytest
import torch

from research_amd.inference import Attention, CacheConfig, FlexAttentionBackend, HipPagedAttentionBackend
from research_amd.inference import InferenceContext


def _cfg(**kw):
    base = dict(num_layers=2, num_kv_heads=4, head_dim=32, num_blocks=16, block_size=4, device="cpu")
    base.update(kw)
    return CacheConfig(**base)


def test_cache_config_surface():
    cfg = CacheConfig(num_layers=3, num_kv_heads=8, head_dim=128)
    assert (cfg.num_blocks, cfg.block_size, cfg.sliding_window, cfg.dtype, cfg.device) == (
        1024, 16, None, torch.bfloat16, "cuda")
    assert cfg.total_slots == 16384 and cfg.cache_shape == (3, 16384, 8, 128)
    # config.py:47-58 of the reference hashes exactly this tuple
    assert hash(cfg) == hash((3, 8, 128, 1024, 16, None, "torch.bfloat16", "cuda"))
    assert cfg == CacheConfig(num_layers=3, num_kv_heads=8, head_dim=128)
    with pytest.raises(Exception):
        cfg.num_layers = 4


def test_backend_attributes_match_reference_surface():
    be = HipPagedAttentionBackend(_cfg())
    # the reference's name: the same class with the reference's decode numerics as defaults
    assert issubclass(FlexAttentionBackend, HipPagedAttentionBackend)
    ref = FlexAttentionBackend(_cfg())
    assert ref.pad_zero_keys and not ref.window_in_decode
    assert not be.pad_zero_keys and be.window_in_decode
    assert be.num_heads_per_kv == 1 and be.scale == 32**-0.5
    assert be.k_cache.shape == (2, 64, 4, 32) and be.k_cache.dtype == torch.bfloat16
    assert not be.k_cache.any() and not be.v_cache.any()
    be.set_num_heads(9)
    assert be.num_heads_per_kv == 2  # integer division, as the reference
    assert be.get_block_mask(2, 8) is None
    be.clear_mask_cache()
    be.k_cache[0, 0] = 1
    be.clear_cache()
    assert not be.k_cache.any()
    for name in ("forward", "_store_kv", "_prefill_attention", "_decode_attention", "_gather_kv_from_cache"):
        assert callable(getattr(be, name))


def test_decode_error_conventions():
    be = HipPagedAttentionBackend(_cfg())
    be.set_num_heads(8)
    q2 = torch.zeros(1, 2, 8, 32, dtype=torch.bfloat16)
    ctx = InferenceContext(is_prefill=False, block_tables=((0,),), seq_lens=(1,))
    with pytest.raises(AssertionError):  # flex_backend.py:199
        be._decode_attention(q2, 0, ctx)
    q1 = q2[:, :1]
    with pytest.raises(ValueError, match="Decode requires block_tables and seq_lens"):  # :201-202
        be._decode_attention(q1, 0, InferenceContext(is_prefill=False))
    with pytest.raises(NotImplementedError):
        be._decode_attention(q1, 0, InferenceContext(is_prefill=False, block_tables=((0,),), seq_lens=(1,),
                                                     block_mask=object()))


def test_mask_objects():
    """The factory functions keep the reference's names and arguments (attention/mask.py) and describe the
    same predicate: mask_mod is compared entry by entry with the range form the kernels receive."""
    from research_amd.inference.attention import (create_attention_mask, create_causal_block_mask,
                                                  create_document_mask, create_sliding_window_causal_mask)
    import numpy as np

    causal = create_causal_block_mask(2, 12, block_size=128, device="cpu")
    swa = create_sliding_window_causal_mask(2, 12, window_size=5)
    assert create_attention_mask(2, 12, sliding_window=None) == causal
    assert create_attention_mask(2, 12, sliding_window=5) == swa
    docs = create_document_mask(1, (3, 0, 4, 2), 12)  # an empty document, and 3 positions past the last one
    assert docs.boundaries == (0, 3, 3, 7, 9) and docs.kind == "document"
    assert (causal.kind, swa.kind) == ("causal", "sliding_window")
    with pytest.raises(ValueError):
        create_sliding_window_causal_mask(1, 8, 0)
    for mask in (causal, swa, docs):
        first = np.maximum(mask.first_keys(np.arange(12)),
                           np.arange(12) - (mask.window or 12) + 1).clip(min=0)
        for qi in range(12):
            for ki in range(12):
                assert mask.mask_mod(0, 0, qi, ki) == (first[qi] <= ki <= qi), (mask.kind, qi, ki)
    assert docs.first_keys(np.arange(12)).tolist() == [0, 0, 0, 3, 3, 3, 3, 7, 7, 9, 9, 9]
    be = HipPagedAttentionBackend(_cfg())
    be.set_num_heads(8)
    q1 = torch.zeros(1, 1, 8, 32, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError, match="document"):
        be._decode_attention(q1, 0, InferenceContext(is_prefill=False, block_tables=((0,),), seq_lens=(1,),
                                                     block_mask=docs))


def test_store_kv_error_conventions():
    be = HipPagedAttentionBackend(_cfg())
    k = torch.zeros(1, 4, 4, 32, dtype=torch.bfloat16)
    with pytest.raises(IndexError, match="shape of the mask"):
        be._store_kv(k, k, 0, (0, 1, 2))
    with pytest.raises(RuntimeError, match="dtypes match"):
        be._store_kv(k.float(), k.float(), 0, (0, 1, 2, 3))
    be._store_kv(k[:, :0], k[:, :0], 0, ())  # nothing to store, no device needed


def test_no_cpu_execution_path():
    """Tensors on the CPU must raise; there is nothing to fall back to."""
    be = HipPagedAttentionBackend(_cfg())
    be.set_num_heads(8)
    k = torch.zeros(1, 4, 4, 32, dtype=torch.bfloat16)
    q = torch.zeros(1, 4, 8, 32, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="HIP device"):
        be._store_kv(k, k, 0, (0, 1, 2, 3))
    with pytest.raises(RuntimeError, match="HIP device"):
        be.forward(q, k, k, 0, InferenceContext(is_prefill=True))
    with pytest.raises(RuntimeError, match="HIP device"):
        be.forward(q[:, :1], k[:, :1], k[:, :1], 0,
                   InferenceContext(is_prefill=False, block_tables=((0,),), seq_lens=(1,)))
    with pytest.raises(RuntimeError, match="HIP device"):
        be._gather_kv_from_cache(0, ((0,),), (3,))


def test_out_of_range_slot_is_an_index_error():
    be = HipPagedAttentionBackend(_cfg())
    k = torch.zeros(1, 2, 4, 32, dtype=torch.bfloat16)
    with pytest.raises(IndexError, match="out of bounds"):
        be._store_kv(k, k, 0, (0, 64))


def test_unsupported_features_raise():
    be = HipPagedAttentionBackend(_cfg(sliding_window=4))
    mask = be.get_block_mask(1, 8)  # a description of the window, cached per shape (flex_backend.py:47-83)
    assert mask.kind == "sliding_window" and mask.window == 4 and be.get_block_mask(1, 8) is mask
    be.clear_mask_cache()
    assert be.get_block_mask(1, 8) is not mask
    with pytest.raises(ValueError):
        HipPagedAttentionBackend(_cfg(sliding_window=0))
    with pytest.raises(ValueError):
        HipPagedAttentionBackend(_cfg(sliding_window=4), pad_zero_keys=True)
    assert HipPagedAttentionBackend(_cfg(sliding_window=4), pad_zero_keys=True, window_in_decode=False)
    with pytest.raises(ValueError):
        HipPagedAttentionBackend(_cfg(kv_format="int4"))
    with pytest.raises(ValueError):
        HipPagedAttentionBackend(_cfg(dtype=torch.float64))


def test_fp8_pool_layout():
    be = HipPagedAttentionBackend(_cfg(kv_format="fp8_e4m3"))
    assert be.k_cache.dtype == torch.float8_e4m3fn and be.k_cache.shape == (2, 64, 4, 32)
    assert be.k_scale.shape == (2, 16, 4) and be.k_scale.dtype == torch.float32 and (be.v_scale == 1).all()


def test_attention_layer_delegates():
    calls = []

    class Probe:
        def forward(self, q, k, v, layer_idx, ctx):
            calls.append((layer_idx, ctx))
            return q

    layer = Attention(layer_idx=3, backend=Probe())
    ctx = InferenceContext(is_prefill=True)
    x = torch.zeros(1)
    assert layer(x, x, x, ctx) is x and calls == [(3, ctx)]
    assert list(layer.parameters()) == []


def test_gather_output_arguments_are_checked_before_any_launch():
    """kv_gather(out=...) validates shape, type and layout on the host; nothing is launched for a bad pair."""
    from research_amd import ops

    pool = torch.zeros((32, 2, 8), dtype=torch.float32)
    tables = torch.zeros((2, 2), dtype=torch.int32)
    lens = torch.tensor([5, 7], dtype=torch.int32)
    good = torch.empty((2, 7, 2, 8), dtype=torch.float32)
    for bad in (torch.empty((2, 6, 2, 8)), torch.empty((2, 7, 2, 8), dtype=torch.float16),
                torch.empty((2, 7, 8, 2)).transpose(2, 3)):
        with pytest.raises(ValueError, match="out tensors"):
            ops.kv_gather(pool, pool, tables, lens, 7, 16, out=(good, bad))


def test_engine_config_defaults():
    from research_amd.inference import EngineConfig

    cfg = EngineConfig(model_path="x")
    assert cfg.cache_type == "none" and cfg.block_size == 16 and cfg.use_graphs is False  # types.py:14-24 + added


def test_prefill_passes():
    """Host logic of the engine's prefill: one pass, or uncached rows first and cached rows second."""
    from research_amd.inference.engine import prefill_passes

    # 2 prompts x 4 rollouts: one full row and three one-token rows each
    cached = [0, 63, 63, 63, 0, 47, 47, 47]
    chunks = [64, 1, 1, 1, 48, 1, 1, 1]
    assert prefill_passes(cached, chunks) == [[0, 4], [1, 2, 3, 5, 6, 7]]
    # nothing cached, or everything cached: one pass in admission order
    assert prefill_passes([0, 0, 0], [5, 9, 2]) == [[0, 1, 2]]
    assert prefill_passes([16, 32], [3, 1]) == [[0, 1]]
    # splitting would not remove enough padding (chunks of similar length): one pass
    assert prefill_passes([0, 16, 0, 16], [40, 30, 38, 35]) == [[0, 1, 2, 3]]
    assert prefill_passes([], []) == [[]]


def test_pack_mask_bit_layout():
    """Bit j of word j // 32 is keep[..., j] (two's-complement int32 words), for key counts around word
    boundaries, broadcast (stride 0) head dimensions and many rows."""
    from research_amd import ops

    g = torch.Generator().manual_seed(3)
    for rows, heads, keys in [(1, 1, 1), (3, 2, 31), (4, 1, 32), (5, 3, 33), (2, 2, 100), (7, 1, 0)]:
        keep = torch.rand((rows, heads, keys), generator=g) < 0.5
        words = ops.pack_mask(keep)
        assert words.dtype == torch.int32 and tuple(words.shape) == (rows, heads, max(1, -(-keys // 32)))
        for r in range(rows):
            for h in range(heads):
                for w in range(words.shape[2]):
                    want = sum(1 << j for j in range(32) if w * 32 + j < keys and keep[r, h, w * 32 + j])
                    assert int(words[r, h, w]) & 0xFFFFFFFF == want
    shared = (torch.rand((6, 1, 64), generator=g) < 0.5).expand(6, 4, 64)
    assert torch.equal(ops.pack_mask(shared), ops.pack_mask(shared.contiguous()))
    tall = torch.rand((70000, 1, 64), generator=g) < 0.5
    words = ops.pack_mask(tall)
    for r in (0, 32767, 32768, 69999):
        want = sum(1 << j for j in range(32) if tall[r, 0, j])
        assert int(words[r, 0, 0]) & 0xFFFFFFFF == want
