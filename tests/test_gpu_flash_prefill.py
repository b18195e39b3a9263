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
    (1, 16, 2, 64, 4100, torch.bfloat16, 0),   # short chunk over a deep prefix: key-range splits + merge
    (1, 8, 2, 33, 3000, torch.float16, 7),
    # odd numbers of 32-row blocks under the late/early pairing of blocks inside a workgroup
    (1, 16, 2, 96, 40, torch.bfloat16, 0),     # 8 heads per KV head, 3 blocks
    (1, 8, 2, 200, 17, torch.float16, 0),      # 4 heads per KV head, 7 blocks
    (1, 4, 2, 150, 70, torch.bfloat16, 2),     # 2 heads per KV head, 5 blocks (two per group)
    (1, 2, 2, 420, 5, torch.bfloat16, 0),      # 1 head per KV head, 14 blocks (four per group)
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


def test_flash_prefill_full_size_sampled_rows():
    """BASELINE config 2 at full size (4096 new tokens over a 32768-token prefix, 16 query / 2 KV heads):
    sampled query rows (block boundaries, first, last) against the oracle run on that one row, 2e-3."""
    from moespresso_amd.runtime.qwen import kquant

    L, past, Hq, Hkv = 4096, 32768, 16, 2
    g = torch.Generator().manual_seed(11)
    q = (0.5 * torch.randn((1, Hq, L, 256), generator=g)).to(torch.bfloat16)
    k = (0.5 * torch.randn((1, Hkv, past + L, 256), generator=g)).to(torch.bfloat16)
    v = (0.5 * torch.randn((1, Hkv, past + L, 256), generator=g)).to(torch.bfloat16)
    scale = 256 ** -0.5
    got = kquant.flash_prefill(q.to(_dev()), k.to(_dev()), v.to(_dev()), scale, past_len=past).float().cpu().numpy()
    kf, vf = k.float().numpy(), v.float().numpy()
    for row in (0, 31, 32, 2047, 2048, 2079, 4064, 4095):
        n = past + row + 1
        want = qwen.causal_prefill_attention(q[:, :, row:row + 1].float().numpy(), kf[:, :, :n], vf[:, :, :n],
                                             scale, past=past + row)
        err = np.abs(got[:, :, row:row + 1] - want)
        assert (err <= 2e-3 + 2.0 ** -8 * np.abs(want)).all(), (row, err.max())


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


def _q8_inputs(past, L, seed, sb_dtype=torch.float32, Hq=16, Hkv=2, B=1):
    """The reference test's recipe (tests/test_qwen_flash_prefill_attention.py:378-388): 0.1 * N(0,1) float32."""
    rng = np.random.default_rng(seed)
    q = (0.1 * rng.standard_normal((B, Hq, L, 256))).astype(np.float32)
    pk = (0.1 * rng.standard_normal((B, Hkv, past, 256))).astype(np.float32)
    pv = (0.1 * rng.standard_normal((B, Hkv, past, 256))).astype(np.float32)
    sk = (0.1 * rng.standard_normal((B, Hkv, L, 256))).astype(np.float32)
    sv = (0.1 * rng.standard_normal((B, Hkv, L, 256))).astype(np.float32)
    out = {}
    for name, x in (("k", pk), ("v", pv)):
        wq, sc, bi = qwen.affine_q8_quantize(x)
        sc_t, bi_t = torch.from_numpy(sc).to(sb_dtype), torch.from_numpy(bi).to(sb_dtype)
        out[name] = (wq, sc_t, bi_t, qwen.affine_q8_dequantize(wq, sc_t.float().numpy(), bi_t.float().numpy()))
    # the caller passes the chunk through the same round trip (full_attention.py:364-369)
    sk_rt = qwen.affine_q8_dequantize(*qwen.affine_q8_quantize(sk))
    sv_rt = qwen.affine_q8_dequantize(*qwen.affine_q8_quantize(sv))
    return q, out["k"], out["v"], sk_rt, sv_rt


@pytest.mark.parametrize("past,L,sb_dtype,self_dtype", [
    (0, 70, torch.float32, torch.float32),
    (64, 48, torch.float32, torch.float32),
    (2065, 135, torch.float32, torch.float32),
    (77, 33, torch.bfloat16, torch.bfloat16),
    (1024, 256, torch.float16, torch.float32),
    (31, 1, torch.float32, torch.float32),
    (4133, 40, torch.float32, torch.float32),   # key-range splits over the quantised prefix
    (6000, 256, torch.bfloat16, torch.float32),
    (700, 1100, torch.bfloat16, torch.float32),   # long chunk: the prefix is converted to float16 rows first
    (45, 1024, torch.float32, torch.bfloat16),
])
def test_sdpa_fa_prefill_q8_matches_oracle(past, L, sb_dtype, self_dtype):
    """Tolerance 1e-2 max-abs (8-bit KV bar) vs float64 attention over the dequantised prefix + chunk."""
    from moespresso_amd.runtime.qwen import kquant

    q, kq8, vq8, sk, sv = _q8_inputs(past, L, seed=past + L, sb_dtype=sb_dtype)
    dev = _dev()

    def words(w):
        return torch.from_numpy(np.ascontiguousarray(w).view(np.int32)).to(dev).view(torch.uint32)

    sk_t, sv_t = torch.from_numpy(sk).to(self_dtype), torch.from_numpy(sv).to(self_dtype)
    scale = 256 ** -0.5
    got = kquant.sdpa_fa_prefill_q8(torch.from_numpy(q).to(dev), words(kq8[0]), kq8[1].to(dev), kq8[2].to(dev),
                                    words(vq8[0]), vq8[1].to(dev), vq8[2].to(dev), sk_t.to(dev), sv_t.to(dev), scale,
                                    bq=32, bk=16, stage=2)
    assert got.dtype == torch.float32 and tuple(got.shape) == q.shape
    k_all = np.concatenate([kq8[3], sk_t.float().numpy()], axis=2)
    v_all = np.concatenate([vq8[3], sv_t.float().numpy()], axis=2)
    want = qwen.causal_prefill_attention(q, k_all, v_all, scale, past=past)
    err = np.abs(got.cpu().numpy() - want).max()
    assert err < 1e-2, err
    # observed accuracy is far inside the bar: 16-bit staging (float16 next to a prefix unpacked in the kernel,
    # bfloat16 for chunks of 1024 queries and more) of values of magnitude 0.1
    assert err < 2e-3, err


def test_sdpa_fa_prefill_q8_full_size_sampled_rows():
    """The reference test's depth (4096 new tokens over a 32768-token 8-bit prefix): sampled query rows against
    the oracle run on that one row over the dequantised prefix + chunk, 1e-2 (8-bit KV bar)."""
    from moespresso_amd.runtime.qwen import kquant

    L, past = 4096, 32768
    q, kq8, vq8, sk, sv = _q8_inputs(past, L, seed=5, sb_dtype=torch.float32)
    dev = _dev()

    def words(w):
        return torch.from_numpy(np.ascontiguousarray(w).view(np.int32)).to(dev).view(torch.uint32)

    scale = 256 ** -0.5
    got = kquant.sdpa_fa_prefill_q8(torch.from_numpy(q).to(dev), words(kq8[0]), kq8[1].to(dev), kq8[2].to(dev),
                                    words(vq8[0]), vq8[1].to(dev), vq8[2].to(dev), torch.from_numpy(sk).to(dev),
                                    torch.from_numpy(sv).to(dev), scale, bq=32, bk=16, stage=2).cpu().numpy()
    k_all = np.concatenate([kq8[3], sk], axis=2)
    v_all = np.concatenate([vq8[3], sv], axis=2)
    for row in (0, 31, 32, 2048, 4095):
        n = past + row + 1
        want = qwen.causal_prefill_attention(q[:, :, row:row + 1], k_all[:, :, :n], v_all[:, :, :n], scale,
                                             past=past + row)
        err = np.abs(got[:, :, row:row + 1] - want).max()
        assert err < 1e-2, (row, err)



def test_sdpa_fa_prefill_q8_chunk_values_beyond_float16_range_saturate():
    """The chunk's own K/V rows are staged as float16: values beyond +-65504 saturate there instead of turning
    into inf (which would make every output row that attends them NaN). Rows inside the range are unaffected."""
    from moespresso_amd.runtime.qwen import kquant

    dev = _dev()
    g = torch.Generator().manual_seed(9)
    L = 40
    q = torch.randn((1, 16, L, 256), generator=g) * 0.1
    sk = torch.randn((1, 2, L, 256), generator=g)
    sv = torch.randn((1, 2, L, 256), generator=g)
    sv[:, :, 7, :8] = 3.0e5                      # one value row far beyond the float16 range
    empty_w = torch.zeros((1, 2, 0, 64), dtype=torch.int32).view(torch.uint32).to(dev)
    empty_s = torch.zeros((1, 2, 0, 4)).to(dev)
    got = kquant.sdpa_fa_prefill_q8(q.to(dev), empty_w, empty_s, empty_s, empty_w, empty_s, empty_s, sk.to(dev),
                                    sv.to(dev), 256 ** -0.5).cpu()
    assert torch.isfinite(got).all()
    want = qwen.causal_prefill_attention(q.numpy(), sk.numpy(), sv.clamp(-65504.0, 65504.0).numpy(), 256 ** -0.5,
                                         past=0)
    err = np.abs(got.numpy() - want)
    assert err[..., 8:].max() < 2e-3 and (err[..., :8] <= 2.0 ** -10 * np.abs(want[..., :8]) + 2e-3).all()
