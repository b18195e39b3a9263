"""GPU parity: causal chunked-prefill attention (through the C-ABI) vs the float64 oracle.

Tolerance: max-abs 2e-3 against float64 softmax attention on the same 16-bit inputs (the bar for
16-bit attention), plus one output ulp where outputs reach magnitude 1.
"""

import numpy as np
import pytest
import torch

from oracle import qwen

pytestmark = pytest.mark.gpu


def _dev():
    return torch.device("cuda:0")


def _case(B, Hq, Hkv, L, past, dtype, seed, extra_rows=0):
    g = torch.Generator().manual_seed(seed)
    q = (0.5 * torch.randn((B, Hq, L, 256), generator=g)).to(dtype)
    k = (0.5 * torch.randn((B, Hkv, past + L + extra_rows, 256), generator=g)).to(dtype)
    v = (0.5 * torch.randn((B, Hkv, past + L + extra_rows, 256), generator=g)).to(dtype)
    return q, k, v


@pytest.mark.parametrize("B,Hq,Hkv,L,past,dtype,extra", [
    (1, 16, 2, 64, 0, torch.bfloat16, 0),
    (1, 16, 2, 32, 96, torch.bfloat16, 0),
    (1, 16, 2, 100, 37, torch.bfloat16, 5),
    (2, 8, 2, 65, 130, torch.float16, 0),
    (1, 4, 2, 1, 300, torch.bfloat16, 0),
    (1, 2, 2, 257, 31, torch.float16, 3),
    (1, 16, 2, 256, 2048, torch.bfloat16, 0),
])
def test_flash_prefill_matches_oracle(B, Hq, Hkv, L, past, dtype, extra):
    from moespresso_amd.runtime.qwen import kquant

    q, k, v = _case(B, Hq, Hkv, L, past, dtype, seed=L + past, extra_rows=extra)
    scale = 256 ** -0.5
    got = kquant.flash_prefill(q.to(_dev()), k.to(_dev()), v.to(_dev()), scale, past_len=past)
    assert got.dtype == dtype and tuple(got.shape) == (B, Hq, L, 256)
    n = past + L
    for b in range(B):
        want = qwen.causal_prefill_attention(q[b:b + 1].float().numpy(), k[b:b + 1, :, :n].float().numpy(),
                                             v[b:b + 1, :, :n].float().numpy(), scale, past=past)
        ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        err = np.abs(got[b:b + 1].float().cpu().numpy() - want)
        assert (err <= 2e-3 + ulp * np.abs(want)).all(), err.max()


def test_flash_prefill_first_row_copies_v():
    """With no prefix the first query row sees one key: its output is that key's V row exactly."""
    from moespresso_amd.runtime.qwen import kquant

    q, k, v = _case(1, 16, 2, 40, 0, torch.bfloat16, seed=3)
    got = kquant.flash_prefill(q.to(_dev()), k.to(_dev()), v.to(_dev()), 0.0625, past_len=0).cpu()
    for h in range(16):
        assert torch.equal(got[0, h, 0], v[0, h // 8, 0])


def test_flash_prefill_validation():
    from moespresso_amd.runtime.qwen import kquant

    dev = _dev()
    q = torch.zeros((1, 16, 8, 256), device=dev, dtype=torch.bfloat16)
    kv = torch.zeros((1, 2, 8, 256), device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="past_len"):
        kquant.flash_prefill(q, kv, kv, 1.0, past_len=1)
    with pytest.raises(ValueError, match="1, 2, 4 or 8"):
        kquant.flash_prefill(q, kv[:, :1], kv[:, :1], 1.0, past_len=0)
    with pytest.raises(ValueError, match="float16 or bfloat16"):
        kquant.flash_prefill(q.float(), kv, kv, 1.0, past_len=0)
