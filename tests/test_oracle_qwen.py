"""Pins for the Qwen/Ornith half of the CPU oracle (no GPU needed)."""

import numpy as np
import torch

from oracle import qwen


def test_gqa_decode_matches_torch_sdpa_float64():
    rng = np.random.default_rng(0)
    q = rng.standard_normal((2, 8, 1, 32))
    k = rng.standard_normal((2, 2, 50, 32))
    v = rng.standard_normal((2, 2, 50, 32))
    got = qwen.gqa_decode_attention(q, k, v, 32 ** -0.5)
    tq, tk, tv = (torch.from_numpy(a) for a in (q, k, v))
    want = torch.nn.functional.scaled_dot_product_attention(
        tq, tk.repeat_interleave(4, 1), tv.repeat_interleave(4, 1), scale=32 ** -0.5).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)


def test_causal_prefill_matches_torch_masked_softmax():
    rng = np.random.default_rng(1)
    past, tq, d = 37, 19, 16
    q = rng.standard_normal((1, 4, tq, d))
    k = rng.standard_normal((1, 2, past + tq, d))
    v = rng.standard_normal((1, 2, past + tq, d))
    got = qwen.causal_prefill_attention(q, k, v, d ** -0.5, past=past, q_chunk=7)
    mask = torch.ones(tq, past + tq, dtype=torch.bool).tril(diagonal=past)
    want = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q), torch.from_numpy(k).repeat_interleave(2, 1),
        torch.from_numpy(v).repeat_interleave(2, 1), attn_mask=mask, scale=d ** -0.5).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)
    # first query row sees exactly past+1 keys
    s = (q[0, 0, 0] @ k[0, 0, :past + 1].T) * d ** -0.5
    p = np.exp(s - s.max())
    np.testing.assert_allclose(got[0, 0, 0], (p / p.sum()) @ v[0, 0, :past + 1], rtol=1e-10)


def test_affine_q8_round_trip_and_packing():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((3, 5, 256)).astype(np.float32)
    packed, scales, biases = qwen.affine_q8_quantize(x)
    assert packed.shape == (3, 5, 64) and packed.dtype == np.dtype("<u4")
    assert scales.shape == (3, 5, 4) and biases.shape == (3, 5, 4)
    deq = qwen.affine_q8_dequantize(packed, scales, biases)
    span = (x.reshape(3, 5, 4, 64).max(-1) - x.reshape(3, 5, 4, 64).min(-1))
    err = np.abs(deq - x).reshape(3, 5, 4, 64).max(-1)
    # the rescaled step (edge / round(edge/scale)) lets the far edge clip by < one step
    assert np.all(err <= span / 255.0 + 1e-6)
    # element j of each word lives in bits [8j, 8j+8)
    codes = np.clip(np.rint((x.reshape(3, 5, 4, 64) - biases[..., None]) / scales[..., None]), 0, 255)
    codes = codes.reshape(3, 5, 256).astype(np.uint32)
    for j in range(4):
        np.testing.assert_array_equal((packed >> (8 * j)) & 0xFF, codes[..., j::4])
    # constant groups survive
    c = np.full((1, 64), 0.75, dtype=np.float32)
    np.testing.assert_allclose(qwen.affine_q8_dequantize(*qwen.affine_q8_quantize(c)), c, atol=1e-6)


def test_q8_0_round_trip():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 256)).astype(np.float32)
    codes, scales = qwen.q8_0_quantize(x)
    assert codes.dtype == np.int8 and scales.dtype == np.float16 and scales.shape == (4, 8)
    deq = qwen.q8_0_dequantize(codes, scales)
    amax = np.abs(x.reshape(4, 8, 32)).max(-1, keepdims=True)
    err = np.abs(deq - x).reshape(4, 8, 32)
    # half a code step plus the float16 rounding of the scale
    assert np.all(err <= amax / 127.0 * 0.5 + amax * 2.0 ** -10)
    assert np.abs(codes).max() <= 127
    z = np.zeros((1, 32), dtype=np.float32)
    np.testing.assert_array_equal(qwen.q8_0_dequantize(*qwen.q8_0_quantize(z)), z)
