"""Eligibility and gates of the fused rope seam (no GPU): the reference's
tests/test_deepseek_v4_attention_seam_kernel.py:166-192, :210-243, :259-270 on torch tensors."""

import torch

from moespresso_amd.runtime.deepseek_v4 import attention_seam_kernel as seam


def test_prefill_rope_seam_gate_and_row_caps(monkeypatch):
    inv_freq = torch.zeros((32,), dtype=torch.float32)
    prefill_shaped = torch.zeros((1, 64, 2, 512), dtype=torch.float32)
    monkeypatch.delenv(seam._PREFILL_ENV_FLAG, raising=False)
    assert seam.prefill_rope_seam_enabled()
    assert seam.partial_rope_eligible(prefill_shaped, inv_freq, offset=0, positions=None)
    monkeypatch.setenv(seam._PREFILL_ENV_FLAG, "0")
    assert not seam.prefill_rope_seam_enabled()
    assert not seam.partial_rope_eligible(prefill_shaped, inv_freq, offset=0, positions=None)
    assert seam.partial_rope_eligible(torch.zeros((1, 64, 1, 512)), inv_freq, offset=0, positions=None)
    monkeypatch.delenv(seam._PREFILL_ENV_FLAG, raising=False)
    monkeypatch.setattr(seam, "_MAX_ROWS_PREFILL", 100)
    assert not seam.partial_rope_eligible(prefill_shaped, inv_freq, offset=0, positions=None)


def test_partial_rope_eligibility_fails_closed():
    inv_freq = torch.zeros((32,), dtype=torch.float32)
    good = torch.zeros((1, 64, 1, 512), dtype=torch.float32)
    assert seam.partial_rope_eligible(good, inv_freq, offset=0, positions=None)
    assert seam.partial_rope_eligible(good, inv_freq, offset=0, positions=torch.zeros((1,)))
    checks = [
        (torch.zeros((1, 1, 1, 32)), inv_freq, 0, None),                      # width below the rope tail
        (torch.zeros((1, 1, 1, 66)), inv_freq, 0, None),                      # width not a multiple of 4
        (torch.zeros((1, 1, 1, 512), dtype=torch.int32), inv_freq, 0, None),  # element dtype
        (good, inv_freq, 1 << 24, None),                                      # beyond float32's exact integers
        (good, inv_freq, -1, None),                                           # negative offset
        (good, inv_freq, 3.5, None),                                          # non-integer offset
        (good, inv_freq.to(torch.float16), 0, None),                          # inv_freq dtype
        (good, torch.zeros((16,)), 0, None),                                  # inv_freq width
        (good, inv_freq, 0, torch.zeros((1,), dtype=torch.float16)),          # positions dtype
        (good, inv_freq, 0, torch.zeros((2,))),                               # positions length
        (good, inv_freq, 0, [0.0]),                                           # positions of a non-tensor type
    ]
    for x, freqs, offset, positions in checks:
        assert not seam.partial_rope_eligible(x, freqs, offset=offset, positions=positions)


def test_rope_seam_gates(monkeypatch):
    monkeypatch.setattr(seam, "_metal_available", lambda: True)
    monkeypatch.delenv(seam._FAMILY_ENV_FLAG, raising=False)
    monkeypatch.delenv(seam._ROPE_ENV_FLAG, raising=False)
    assert seam.rope_seam_enabled()
    monkeypatch.setenv(seam._FAMILY_ENV_FLAG, "0")
    assert not seam.rope_seam_enabled()
    monkeypatch.delenv(seam._FAMILY_ENV_FLAG)
    monkeypatch.setenv(seam._ROPE_ENV_FLAG, "0")
    assert not seam.rope_seam_enabled()
    monkeypatch.delenv(seam._ROPE_ENV_FLAG)
    monkeypatch.setattr(seam, "_metal_available", lambda: False)
    assert not seam.rope_seam_enabled()


def test_cpu_operands_are_refused_loudly():
    import pytest
    with pytest.raises(RuntimeError, match="HIP device"):
        seam.fused_partial_rope(torch.zeros((1, 1, 1, 64)), torch.zeros((32,)), offset=0)
