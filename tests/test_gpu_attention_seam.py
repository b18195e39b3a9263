"""GPU parity: the fused partial rope (through the C-ABI) vs the NumPy oracle, bit for bit.

Shapes, offsets and rope parameter sets follow the reference's
tests/test_deepseek_v4_attention_seam_kernel.py (:60-163); the composed sequence the reference
compares against lives in a third-party package, so the oracle restates the kernel body the reference
ships (attention_seam_kernel.py:80-118) and is pinned on the CPU side against the float64 closed form
and NumPy's native float16 arithmetic.
"""

import numpy as np
import pytest
import torch

from moespresso_amd.runtime.deepseek_v4 import attention_seam_kernel as seam
from oracle import ds4

pytestmark = pytest.mark.gpu

_YARN = {"factor": 16.0, "original_seq_len": 65536, "beta_fast": 32, "beta_slow": 1}
_TORCH = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def _ropes():
    return {"compress_yarn": ds4.rope_inverse_frequencies(64, 160000.0, _YARN).astype(np.float32),
            "swa_plain": ds4.rope_inverse_frequencies(64, 10000.0).astype(np.float32)}


def _rope_input(shape, dtype_name, seed):
    """The reference's _rope_input (:51-55): 2*N(0,1) with about 1 % negative zeros."""
    rng = np.random.default_rng(seed)
    x = (2.0 * rng.standard_normal(shape)).astype(np.float32)
    x[rng.random(shape) < 0.01] = -0.0
    t = torch.from_numpy(x).to(_TORCH[dtype_name])
    return t.to("cuda:0"), t.float().numpy()


def _bits(t):
    t = t.cpu().contiguous()
    return t.view({4: torch.int32, 2: torch.int16}[t.element_size()]).numpy()


def _check(x_dev, x_np, inv, dtype_name, **kw):
    inv_dev = torch.from_numpy(inv).to("cuda:0")
    pos = kw.get("positions")
    got = seam.fused_partial_rope(x_dev, inv_dev, offset=kw.get("offset", 0), inverse=kw.get("inverse", False),
                                  positions=None if pos is None else torch.from_numpy(pos).to("cuda:0"))
    assert got.shape == x_dev.shape and got.dtype == x_dev.dtype
    want = ds4.fused_partial_rope(x_np, inv, offset=kw.get("offset", 0), inverse=kw.get("inverse", False),
                                  positions=pos, dtype=dtype_name)
    want_t = torch.from_numpy(want).to(_TORCH[dtype_name])
    np.testing.assert_array_equal(_bits(got), _bits(want_t))


@pytest.mark.parametrize("dtype_name", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("shape", [(1, 64, 1, 512), (1, 1, 1, 512), (1, 64, 1, 128), (1, 1, 1, 64)])
@pytest.mark.parametrize("inverse", [False, True])
def test_fused_partial_rope_bit_identical(dtype_name, shape, inverse):
    for inv in _ropes().values():
        for offset in (0, 1, 3855, (1 << 24) - 2):
            x_dev, x_np = _rope_input(shape, dtype_name, offset + shape[1] + shape[3])
            _check(x_dev, x_np, inv, dtype_name, offset=offset, inverse=inverse)


@pytest.mark.parametrize("dtype_name", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("rows", [1, 3])
def test_fused_partial_rope_positions_form_bit_identical(dtype_name, rows):
    positions = (np.arange(rows, dtype=np.float32) * 4.0 + 3844.0).astype(np.float32)
    x_dev, x_np = _rope_input((1, 1, rows, 512), dtype_name, rows)
    _check(x_dev, x_np, _ropes()["compress_yarn"], dtype_name, positions=positions)


# served prefill shapes of the reference's census (:110-119), the large ones with fewer rows so that the
# oracle's Python loop over positions stays within seconds
@pytest.mark.parametrize("shape,dtype_name,offset,inverse", [
    ((1, 64, 769, 512), "bfloat16", 0, False),
    ((1, 64, 769, 512), "float32", 0, True),
    ((1, 1, 3843, 512), "float32", 0, False),
    ((1, 64, 769, 128), "float32", 0, False),
    ((1, 64, 311, 512), "bfloat16", 6144, False),
    ((1, 64, 214, 512), "float32", 14336, True),
    ((1, 64, 7, 512), "bfloat16", 4096, False),
    ((2, 3, 7, 512), "float16", 4096, True),
])
def test_fused_partial_rope_prefill_rows_bit_identical(shape, dtype_name, offset, inverse):
    for inv in _ropes().values():
        x_dev, x_np = _rope_input(shape, dtype_name, offset + shape[2] + shape[3])
        _check(x_dev, x_np, inv, dtype_name, offset=offset, inverse=inverse)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("width", [512, 128])
def test_fused_partial_rope_prefill_positions_form_bit_identical(dtype_name, width):
    rows = 960
    positions = (np.arange(rows, dtype=np.float32) * 4.0 + 3.0).astype(np.float32)
    x_dev, x_np = _rope_input((1, 1, rows, width), dtype_name, rows + width)
    _check(x_dev, x_np, _ropes()["compress_yarn"], dtype_name, positions=positions)


def test_full_anchor_chunk_inverse_undoes_forward():
    # the 3843-row anchor chunk at full size: a property instead of the oracle loop
    inv = torch.from_numpy(_ropes()["compress_yarn"]).to("cuda:0")
    x = 2.0 * torch.randn((1, 64, 3843, 512), device="cuda:0", generator=torch.Generator("cuda:0").manual_seed(3))
    y = seam.fused_partial_rope(x, inv, offset=0)
    back = seam.fused_partial_rope(y, inv, offset=0, inverse=True)
    assert torch.equal(y[..., :448], x[..., :448])
    assert float((back - x).abs().max()) < 1e-4
    # norm of every rotated pair is preserved
    n0 = x[..., 448:].reshape(-1, 32, 2).norm(dim=-1)
    n1 = y[..., 448:].reshape(-1, 32, 2).norm(dim=-1)
    assert float((n0 - n1).abs().max()) < 1e-4
    assert ("off", False) in seam._ROPE_KERNELS and ("off", True) in seam._ROPE_KERNELS


def test_fused_partial_rope_raises_outside_contract(monkeypatch):
    inv = torch.zeros((32,), device="cuda:0")
    with pytest.raises(ValueError):
        seam.fused_partial_rope(torch.zeros((1, 64, 1, 32), device="cuda:0"), inv, offset=0)
    monkeypatch.setenv(seam._PREFILL_ENV_FLAG, "0")
    with pytest.raises(ValueError):
        seam.fused_partial_rope(torch.zeros((1, 64, 2, 512), device="cuda:0"), inv, offset=0)
