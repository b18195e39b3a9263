"""NumPy restatement of the Qwen/Ornith side of the attention hot path.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

The arithmetic of this half lives in two un-vendored dependencies of the
reference, neither present in the reference tree:

* ``mlx-kquant 0.3.0 @ e165cafafa149493d298871c610e29e95ffa8f10``
  (``sdpa_decode_q8``, ``sdpa_fa_prefill_q8``; pinned in the reference's
  ``pyproject.toml:12``), called at
  ``src/moespresso/runtime/qwen/full_attention.py:323-335`` and ``:372-382``;
* ``mlx 0.31.2`` (``mx.quantize`` / ``mx.dequantize`` affine 8-bit, group 64;
  ``mx.fast.scaled_dot_product_attention``).

Their published algorithm is restated here: softmax(q K^T scale [+ causal]) V in
float64 over the dequantised cache, query head ``h`` reading KV head
``h // (Hq / Hkv)``. The attention closed form is pinned against
``torch.softmax`` in float64; the affine quantiser's edge rules are restated
from MLX's published ``affine_quantize`` and are "parity unpinned" (no vectors
for them exist in the reference tree). The kernels under test consume
``(codes, scales, biases)`` and only depend on ``code * scale + bias`` and on
the little-endian packing of four codes per 32-bit word.
"""

from __future__ import annotations

import numpy as np

F32 = np.float32


# --------------------------------------------------------------------------
# Q8 KV formats
# --------------------------------------------------------------------------

def affine_q8_quantize(x: np.ndarray, group_size: int = 64):
    """MLX-style affine 8-bit quantisation over the last axis.

    Per group: ``scale = max((max-min)/255, 1e-7)`` signed so that the edge
    with the larger magnitude is represented exactly, ``bias = that edge``;
    ``code = clip(round((x-bias)/scale), 0, 255)``. Returns ``(packed uint32
    [..., D/4], scales f32 [..., D/group], biases f32 [..., D/group])``; four
    codes per word, element ``j`` in bits ``[8j, 8j+8)``.
    (Call-site layout: test_qwen_flash_prefill_attention.py:361-370 of the
    reference; quantiser rule: mlx 0.31.2 ``affine_quantize``. Parity unpinned.)
    """
    x = np.asarray(x, dtype=F32)
    d = x.shape[-1]
    g = x.reshape(*x.shape[:-1], d // group_size, group_size)
    # float32 throughout, one rounding per operation (the order of the Metal kernel's statements)
    w_max = g.max(axis=-1, keepdims=True)
    w_min = g.min(axis=-1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        scales = np.maximum(((w_max - w_min).astype(F32) / F32(255.0)).astype(F32), F32(1e-7))
        side = np.abs(w_min) > np.abs(w_max)
        scales = np.where(side, scales, -scales).astype(F32)
        edge = np.where(side, w_min, w_max).astype(F32)
        q0 = np.rint((edge / scales).astype(F32))
        at_zero = q0 == 0
        scales = np.where(at_zero, scales, (edge / np.where(at_zero, F32(1.0), q0)).astype(F32)).astype(F32)
        biases = np.where(at_zero, F32(0.0), edge).astype(F32)
        codes = np.rint(((g - biases).astype(F32) / scales).astype(F32))
    codes = np.clip(codes, 0, 255).astype(np.uint8).reshape(*x.shape[:-1], d)
    packed = np.ascontiguousarray(codes).view("<u4")
    return packed, scales[..., 0], biases[..., 0]


def affine_q8_dequantize(packed: np.ndarray, scales: np.ndarray, biases: np.ndarray,
                         group_size: int = 64) -> np.ndarray:
    """``code * scale + bias`` in float32 (the in-kernel dequant contract)."""
    codes = np.ascontiguousarray(np.asarray(packed).astype("<u4")).view(np.uint8).astype(F32)
    d = codes.shape[-1]
    g = codes.reshape(*codes.shape[:-1], d // group_size, group_size)
    s = np.asarray(scales, dtype=F32)[..., None]
    b = np.asarray(biases, dtype=F32)[..., None]
    return (g * s + b).astype(F32).reshape(codes.shape)


def q8_0_quantize(x: np.ndarray, block: int = 32):
    """Symmetric int8 blocks with one float16 scale (BASELINE config 3 format).

    ``d = amax/127`` (float32), ``code = clip(round(x/d), -127, 127)``, scale
    stored as float16. Returns ``(int8 [..., D], float16 [..., D/block])``.
    """
    x = np.asarray(x, dtype=F32)
    d = x.shape[-1]
    g = x.reshape(*x.shape[:-1], d // block, block)
    amax = np.max(np.abs(g), axis=-1, keepdims=True)
    scale = (amax / F32(127.0)).astype(F32)
    inv = np.where(scale > 0, F32(1.0) / np.where(scale > 0, scale, F32(1.0)), F32(0.0)).astype(F32)
    codes = np.clip(np.rint(g * inv), -127, 127).astype(np.int8).reshape(x.shape)
    return codes, scale[..., 0].astype(np.float16)


def q8_0_dequantize(codes: np.ndarray, scales: np.ndarray, block: int = 32) -> np.ndarray:
    """``code * float32(scale_f16)`` in float32."""
    c = np.asarray(codes, dtype=np.int8).astype(F32)
    d = c.shape[-1]
    g = c.reshape(*c.shape[:-1], d // block, block)
    return (g * np.asarray(scales).astype(F32)[..., None]).astype(F32).reshape(c.shape)


# --------------------------------------------------------------------------
# attention closed forms
# --------------------------------------------------------------------------

def gqa_decode_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float) -> np.ndarray:
    """One-token GQA attention, float64.

    q ``[B,Hq,1,D]``, k/v ``[B,Hkv,N,D]`` -> ``[B,Hq,1,D]``; head ``h`` reads KV
    head ``h // (Hq/Hkv)`` (full_attention.py:323-335 call site; BASELINE
    configs 1 and 3).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    b, hq, tq, d = q.shape
    hkv = k.shape[1]
    rep = hq // hkv
    out = np.zeros((b, hq, tq, v.shape[-1]), dtype=np.float64)
    for bi in range(b):
        for h in range(hq):
            kh = k[bi, h // rep]
            s = (q[bi, h] @ kh.T) * float(scale)
            s = s - s.max(axis=-1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=-1, keepdims=True)
            out[bi, h] = p @ v[bi, h // rep]
    return out


def causal_prefill_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float,
                             *, past: int, q_chunk: int = 512) -> np.ndarray:
    """Causal GQA prefill with a ``past``-token prefix, float64.

    q ``[1,Hq,Tq,D]``; k/v ``[1,Hkv,past+Tq,D]``: query ``t`` sees keys
    ``[0, past+t]`` (full_attention.py:372-382 call site; BASELINE config 2).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    b, hq, tq, d = q.shape
    hkv = k.shape[1]
    rep = hq // hkv
    n = k.shape[2]
    out = np.zeros((b, hq, tq, v.shape[-1]), dtype=np.float64)
    kidx = np.arange(n)
    for bi in range(b):
        for h in range(hq):
            kh, vh = k[bi, h // rep], v[bi, h // rep]
            for t0 in range(0, tq, q_chunk):
                t1 = min(tq, t0 + q_chunk)
                s = (q[bi, h, t0:t1] @ kh.T) * float(scale)
                mask = kidx[None, :] > (past + np.arange(t0, t1))[:, None]
                s = np.where(mask, -np.inf, s)
                s = s - s.max(axis=-1, keepdims=True)
                p = np.exp(s)
                p /= p.sum(axis=-1, keepdims=True)
                out[bi, h, t0:t1] = p @ vh
    return out
