"""GPU parity: one-token GQA decode over an 8-bit KV cache (through the C-ABI) vs the float64 oracle.

Tolerance: max-abs 1e-2 against float64 softmax attention over the dequantised cache (the bar for
8-bit KV); observed errors are about 1e-3 (float16 staging of K, V and the probabilities).
"""

import numpy as np
import pytest
import torch

from oracle import qwen

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _dev():
    return torch.device("cuda:0")


def _affine_cache(rng, B, Hkv, N, sb_dtype):
    k = rng.standard_normal((B, Hkv, N, 256), dtype=np.float32)
    v = rng.standard_normal((B, Hkv, N, 256), dtype=np.float32)
    kq = qwen.affine_q8_quantize(k)
    vq = qwen.affine_q8_quantize(v)

    def cast(a):
        return torch.from_numpy(a).to(sb_dtype)

    ks, kb, vs, vb = cast(kq[1]), cast(kq[2]), cast(vq[1]), cast(vq[2])
    kd = qwen.affine_q8_dequantize(kq[0], ks.float().numpy(), kb.float().numpy())
    vd = qwen.affine_q8_dequantize(vq[0], vs.float().numpy(), vb.float().numpy())
    dev = _dev()
    args = (torch.from_numpy(kq[0].view(np.int32)).to(dev).view(torch.uint32), ks.to(dev), kb.to(dev),
            torch.from_numpy(vq[0].view(np.int32)).to(dev).view(torch.uint32), vs.to(dev), vb.to(dev))
    return args, kd, vd


@pytest.mark.parametrize("B,Hq,Hkv,N,sb_dtype", [
    (1, 16, 2, 1, torch.float32),
    (1, 16, 2, 31, torch.float32),
    (1, 16, 2, 257, torch.bfloat16),
    (2, 8, 4, 1000, torch.float16),
    (1, 16, 2, 4099, torch.bfloat16),
    (1, 16, 2, 8192, torch.bfloat16),      # the depth from which the reference engages this operator
    (1, 16, 2, 37000, torch.bfloat16),     # BASELINE config 3 depth, scales as served (bfloat16)
    (1, 4, 4, 300, torch.float32),
    (1, 32, 2, 129, torch.float32),
])
def test_sdpa_decode_q8_affine(B, Hq, Hkv, N, sb_dtype):
    from moespresso_amd.runtime.qwen import kquant

    rng = np.random.default_rng(N * 7 + Hq)
    args, kd, vd = _affine_cache(rng, B, Hkv, N, sb_dtype)
    q = rng.standard_normal((B, Hq, 1, 256), dtype=np.float32)
    scale = 256 ** -0.5
    got = kquant.sdpa_decode_q8(torch.from_numpy(q).to(_dev()), *args, scale, group_size=64, bits=8, splits=128,
                                stage=2, compute=1, tile_c=16)
    assert got.dtype == torch.float32 and tuple(got.shape) == (B, Hq, 1, 256)
    want = qwen.gqa_decode_attention(q, kd, vd, scale)
    err = np.abs(got.cpu().numpy() - want).max()
    assert err < TOL, err


@pytest.mark.parametrize("B,N,qdt", [
    (1, 37000, torch.bfloat16),
    (8, 37000, torch.bfloat16),
    (1, 513, torch.float16),
    (3, 2048, torch.float32),
    (3, 37000, torch.bfloat16),   # batch x KV heads does not divide the CU count
    (5, 9000, torch.float16),
])
def test_sdpa_decode_q8_0(B, N, qdt):
    """BASELINE config 3: int8 codes + one float16 scale per 32, bf16 queries, batch 1 and 8."""
    from moespresso_amd.runtime.qwen import kquant

    Hq, Hkv = 16, 2
    rng = np.random.default_rng(B * 100 + N)
    k = rng.standard_normal((B, Hkv, N, 256), dtype=np.float32)
    v = rng.standard_normal((B, Hkv, N, 256), dtype=np.float32)
    kc, ks = qwen.q8_0_quantize(k)
    vc, vs = qwen.q8_0_quantize(v)
    kd, vd = qwen.q8_0_dequantize(kc, ks), qwen.q8_0_dequantize(vc, vs)
    q = torch.from_numpy(rng.standard_normal((B, Hq, 256), dtype=np.float32)).to(qdt)
    scale = 256 ** -0.5
    dev = _dev()
    got = kquant.sdpa_decode_q8_0(q.to(dev), torch.from_numpy(kc).to(dev), torch.from_numpy(ks).to(dev),
                                  torch.from_numpy(vc).to(dev), torch.from_numpy(vs).to(dev), scale)
    assert got.dtype == qdt and tuple(got.shape) == (B, Hq, 256)
    want = qwen.gqa_decode_attention(q.float().numpy()[:, :, None, :], kd, vd, scale)[:, :, 0, :]
    err = np.abs(got.float().cpu().numpy() - want).max()
    assert err < TOL, err


def test_sdpa_decode_q8_one_hot_rows_exact():
    """A query that puts all its weight on one key returns that key's dequantised V row (float16-exact data)."""
    from moespresso_amd.runtime.qwen import kquant

    B, Hq, Hkv, N = 1, 16, 2, 640
    rng = np.random.default_rng(5)
    kc = np.zeros((B, Hkv, N, 256), dtype=np.int8)
    hot = rng.integers(0, N, size=(Hkv,))
    for h in range(Hkv):
        kc[0, h, hot[h], :] = 127
    ks = np.full((B, Hkv, N, 8), 1.0, dtype=np.float16)
    vc = rng.integers(-127, 128, size=(B, Hkv, N, 256)).astype(np.int8)
    vs = np.full((B, Hkv, N, 8), 0.25, dtype=np.float16)
    q = np.full((B, Hq, 256), 1.0, dtype=np.float32)
    dev = _dev()
    got = kquant.sdpa_decode_q8_0(torch.from_numpy(q).to(dev), torch.from_numpy(kc).to(dev),
                                  torch.from_numpy(ks).to(dev), torch.from_numpy(vc).to(dev),
                                  torch.from_numpy(vs).to(dev), 1.0).cpu().numpy()
    for h in range(Hq):
        # the hot key's logit leads by 127*256, every other weight underflows to zero
        np.testing.assert_array_equal(got[0, h], vc[0, h // 8, hot[h // 8]].astype(np.float32) * 0.25)


def test_sdpa_decode_q8_validation():
    from moespresso_amd.runtime.qwen import kquant

    dev = _dev()
    q = torch.zeros((1, 16, 1, 256), device=dev)
    wq = torch.zeros((1, 2, 8, 64), device=dev, dtype=torch.int32).view(torch.uint32)
    sb = torch.zeros((1, 2, 8, 4), device=dev)
    with pytest.raises(ValueError, match="group_size=64, bits=8"):
        kquant.sdpa_decode_q8(q, wq, sb, sb, wq, sb, sb, 1.0, group_size=32, bits=8)
    with pytest.raises(ValueError, match="single-token"):
        kquant.sdpa_decode_q8(torch.zeros((1, 16, 2, 256), device=dev), wq, sb, sb, wq, sb, sb, 1.0)
    with pytest.raises(ValueError, match="float32"):
        kquant.sdpa_decode_q8(q.half(), wq, sb, sb, wq, sb, sb, 1.0)
    with pytest.raises(RuntimeError, match="HIP device"):
        kquant.sdpa_decode_q8(q.cpu(), wq, sb, sb, wq, sb, sb, 1.0)
