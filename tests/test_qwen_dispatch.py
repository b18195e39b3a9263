"""Host logic of the Qwen full-attention dispatch and the DS4 fixed-state helpers (no GPU needed).

Follows the branch/counter tests of the reference's tests/test_qwen_flash_prefill_attention.py.
"""

import types

import numpy as np
import pytest
import torch

from moespresso_amd.runtime.deepseek_v4 import fixed_decode_state as fds
from moespresso_amd.runtime.qwen import full_attention as fa
from moespresso_amd.runtime.qwen import kquant
from oracle import ds4


def _stub_cache(offset=100):
    cache = kquant.QuantizedKVCache(group_size=64, bits=8)
    cache.offset = offset
    cache.keys = object()  # only "is not None" is inspected
    return cache


def _wrapper(kv_heads=2):
    inner = types.SimpleNamespace(num_key_value_heads=kv_heads, num_attention_heads=16)
    return fa.FlashPrefillD256Attention(inner)


def test_flash_eligibility_counts_first_failing_branch(monkeypatch):
    monkeypatch.setattr(fa, "_kernel_available", lambda: True)
    monkeypatch.setattr(fa, "_QWEN_PREFILL_FLASH_D256", True)
    w = _wrapper()
    q = torch.zeros((1, 16, 8, 256))
    assert w._flash_eligible(q, _stub_cache(), "causal")
    assert not w._flash_eligible(q[:, :, :1], _stub_cache(), "causal") and w.fallback_decode == 1
    assert not w._flash_eligible(q, None, "causal") and w.fallback_cache == 1
    assert not w._flash_eligible(q, _stub_cache(offset=0), "causal") and w.fallback_cache == 2
    assert not w._flash_eligible(q, _stub_cache(), None) and w.fallback_mask == 1
    assert not w._flash_eligible(q[:, :8], _stub_cache(), "causal") and w.fallback_geometry == 1
    assert not w._flash_eligible(torch.zeros((2, 16, 8, 256)), _stub_cache(), "causal") and w.fallback_geometry == 2
    assert not _wrapper(kv_heads=4)._flash_eligible(q, _stub_cache(), "causal")
    assert not w._flash_eligible(q.half(), _stub_cache(), "causal") and w.fallback_dtype == 1
    monkeypatch.setattr(fa, "_kernel_available", lambda: False)
    assert not w._flash_eligible(q, _stub_cache(), "causal") and w.fallback_kernel == 1
    monkeypatch.setattr(fa, "_QWEN_PREFILL_FLASH_D256", False)
    assert not w._flash_eligible(q, _stub_cache(), "causal") and w.fallback_prefill_disabled == 1
    assert w.flash_calls == 0


def test_decode_eligibility_and_min_keys(monkeypatch):
    monkeypatch.setattr(fa, "_decode_kernel_available", lambda: True)
    monkeypatch.setattr(fa, "_QWEN_DECODE_Q8_TILE16", True)
    w = _wrapper()
    q = torch.zeros((1, 16, 1, 256))
    assert w._decode_eligible(q, _stub_cache(offset=8191), None)          # 8191 + 1 keys
    assert not w._decode_eligible(q, _stub_cache(offset=8190), None) and w.fallback_decode == 1
    monkeypatch.setattr(fa, "_DECODE_Q8_TILE16_MIN_KEYS", 16)
    assert w._decode_eligible(q, _stub_cache(offset=15), None)
    assert not w._decode_eligible(q, _stub_cache(), "causal") and w.fallback_mask == 1
    assert not w._decode_eligible(q.double(), _stub_cache(), None) and w.fallback_dtype == 1
    monkeypatch.setattr(fa, "_QWEN_DECODE_Q8_TILE16", False)
    assert not w._decode_eligible(q, _stub_cache(), None) and w.fallback_decode == 2


def test_install_is_idempotent_and_stats_aggregate(monkeypatch):
    monkeypatch.setattr(fa, "_kernel_available", lambda: True)
    monkeypatch.setattr(fa, "_decode_kernel_available", lambda: True)
    inner = types.SimpleNamespace(num_key_value_heads=2, num_attention_heads=16)
    layers = [types.SimpleNamespace(is_linear=True, self_attn=None),
              types.SimpleNamespace(is_linear=False, self_attn=inner),
              types.SimpleNamespace(is_linear=False, self_attn=inner),
              types.SimpleNamespace(is_linear=False, self_attn=None)]
    model = types.SimpleNamespace(model=types.SimpleNamespace(layers=layers))
    assert fa.install_flash_prefill_attention(model) == 2
    assert fa.install_flash_prefill_attention(model) == 0
    layers[1].self_attn.flash_calls = 3
    layers[2].self_attn.flash_calls = 4
    layers[2].self_attn.fallback_mask = 1
    stats = fa.flash_prefill_attention_stats(model)
    assert stats["wrapped_layers"] == 2 and stats["flash_calls"] == 7 and stats["fallback_mask"] == 1
    monkeypatch.setattr(fa, "_QWEN_PREFILL_FLASH_D256", False)
    monkeypatch.setattr(fa, "_QWEN_DECODE_Q8_TILE16", False)
    fresh = types.SimpleNamespace(layers=[types.SimpleNamespace(is_linear=False, self_attn=inner)])
    assert fa.install_flash_prefill_attention(fresh) == 0


def test_stage_table_and_flags():
    assert fa._STAGE_CONFIGS["f32"] == (2, 64, 16) and fa._STAGE_CONFIGS["f32w32"] == (2, 32, 16)
    assert (fa._FLASH_N_Q_HEADS, fa._FLASH_N_KV_HEADS, fa._FLASH_HEAD_DIM) == (16, 2, 256)
    assert fa._DECODE_Q8_TILE16_MIN_KEYS == 8192
    assert fa.flash_prefill_enabled() == fa._QWEN_PREFILL_FLASH_D256
    assert kquant.HAS_SDPA_DECODE_Q8_DIMENSION_PARALLEL_MERGE


def test_operators_refuse_cpu_tensors():
    x = torch.zeros((1, 2, 4, 256))
    with pytest.raises(RuntimeError, match="HIP device"):
        kquant.quantize(x)
    with pytest.raises(ValueError, match="group_size=64, bits=8"):
        kquant.quantize(x, group_size=32)
    with pytest.raises(ValueError, match="multiple of the group size"):
        kquant.quantize(torch.zeros((3, 100)))


def test_fixed_decode_state_helpers_match_oracle():
    params = fds.decode_step_params(offset=41, pool_rows=5)
    assert params.dtype == torch.int32
    np.testing.assert_array_equal(params.numpy(), ds4.decode_step_params(41, 5))
    rng = np.random.default_rng(0)
    scores = rng.standard_normal((1, 3, 9)).astype(np.float32)
    got = fds.pad_scores_to_capacity(torch.from_numpy(scores), params).numpy()
    np.testing.assert_array_equal(got, ds4.pad_scores_to_capacity(scores, 5))
    # the reference's call sites pass their array module first (fixed_decode_state.py:186,198 called as
    # decode_step_params(mx, offset=…, pool_rows=…) and pad_scores_to_capacity(mx, scores, params))
    np.testing.assert_array_equal(fds.decode_step_params(torch, offset=41, pool_rows=5).numpy(), params.numpy())
    np.testing.assert_array_equal(fds.pad_scores_to_capacity(torch, torch.from_numpy(scores), params).numpy(), got)
    with pytest.raises(TypeError):
        fds.pad_scores_to_capacity(torch.from_numpy(scores))
    with pytest.raises(ValueError, match="int32"):
        fds.pad_scores_to_capacity(torch.from_numpy(scores), params.float())


def test_row_capacity_of_cache_views():
    from moespresso_amd.runtime.qwen.kquant import _cache_operands, _row_capacity

    buf = torch.zeros((2, 2, 512, 64))
    assert _row_capacity(buf[:, :, :300], 300) == 512          # leading rows of every head
    assert _row_capacity(buf, 512) == 512
    assert _row_capacity(buf[:, :, :300].contiguous(), 300) == 300
    assert _row_capacity(buf[:, :, 5:305], 300) == 512         # same strides from another first row
    assert _row_capacity(buf[:, :1, :300], 300) == 1024        # one head of two: the batch stride is the capacity
    assert _row_capacity(buf[:1, :1, :300], 300) == 300
    assert _row_capacity(buf.transpose(1, 2)[:, :300], 300) is None
    assert _row_capacity(buf[:, :, :300, ::2], 300) is None
    a, b = buf[:, :, :300], torch.zeros((2, 2, 768, 4))[:, :, :300]
    same, rows = _cache_operands((a, a), 300)
    assert rows == 512 and same[0] is a
    mixed, rows = _cache_operands((a, b), 300)                 # capacities differ: dense copies
    assert rows == 300 and all(t.is_contiguous() for t in mixed)
