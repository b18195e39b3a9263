"""8-bit-KV attention operators for the Qwen/Ornith full-attention layers on MI355X.

The reference calls two operators of the third-party ``mlx_kquant`` Metal package from
``src/moespresso/runtime/qwen/full_attention.py``: ``sdpa_decode_q8`` (:323) for one-token decode
and ``sdpa_fa_prefill_q8`` (:372) for chunked causal prefill over a quantised prefix. This module
provides operators of the same names and argument order on HIP tensors. The Metal tuning keywords
of the reference call sites (``splits``, ``stage``, ``compute``, ``tile_c``, ``bq``, ``bk``,
``dimension_parallel_merge``) are accepted and ignored: tiling and the split count are chosen for
the 256 compute units of the device by the library.

Cache layout (the MLX affine quantiser, ``mx.quantize(x, group_size=64, bits=8)``): ``wq`` uint32
``[B, Hkv, N, D/4]`` with four codes per word (lowest byte first), ``scales`` and ``biases``
``[B, Hkv, N, D/64]``; value = code * scale + bias.
"""

from __future__ import annotations

import torch

from moespresso_amd import _lib

_HEAD_DIM = 256

# The decode kernel's range merge always spreads the 256 output columns over the merging waves;
# the flag exists because callers probe for it (reference full_attention.py:146-157).
HAS_SDPA_DECODE_Q8_DIMENSION_PARALLEL_MERGE = True


def _check_q8_triplet(name, wq, scales, biases, batch, n_keys=None):
    if wq.ndim != 4 or scales.ndim != 4 or biases.ndim != 4:
        raise ValueError(f"{name} quantized tensors must be rank-4 [B, Hkv, N, *]")
    if wq.dtype != torch.uint32 and wq.dtype != torch.int32 and wq.dtype != torch.uint8:
        raise ValueError(f"{name} codes must be uint32 words (or their uint8 view)")
    width = int(wq.shape[-1]) * (4 if wq.dtype != torch.uint8 else 1)
    if width != _HEAD_DIM:
        raise ValueError("q8 attention requires head_dim=256")
    if int(scales.shape[-1]) != _HEAD_DIM // 64 or tuple(scales.shape) != tuple(biases.shape):
        raise ValueError(f"{name} scales and biases must be [B, Hkv, N, 4] (group_size=64)")
    if scales.dtype != biases.dtype or scales.dtype not in _lib.DTYPE_CODE:
        raise ValueError(f"{name} scales and biases must share a float32/float16/bfloat16 dtype")
    if tuple(wq.shape[:3]) != tuple(scales.shape[:3]) or int(wq.shape[0]) != batch:
        raise ValueError(f"{name} codes, scales and biases disagree on [B, Hkv, N]")
    if n_keys is not None and int(wq.shape[2]) != n_keys:
        raise ValueError("keys and values disagree on the number of cached tokens")


def _row_capacity(t, n_rows: int):
    """Row capacity of a ``[B, H, n_rows, W]`` tensor that is the first ``n_rows`` rows of every head of a
    dense ``[B, H, capacity, W]`` buffer (what a cache that grows in blocks hands out), else ``None``."""
    B, H, N, W = (int(v) for v in t.shape)
    sb, sh, sn, sw = (int(v) for v in t.stride())
    if sw != 1 or sn != W:
        return None
    if B * H == 1:
        return N
    cap = (sh if H > 1 else sb) // W if W else 0
    if cap < N or (H > 1 and sh != cap * W) or (B > 1 and sb != H * cap * W):
        return None
    return cap


def _cache_operands(tensors, n_rows: int):
    """The cache tensors as the library reads them: untouched when all of them are leading-row views of dense
    buffers with one common row capacity (no copy), otherwise dense copies with capacity ``n_rows``."""
    caps = [_row_capacity(t, n_rows) for t in tensors]
    if caps[0] is not None and all(c == caps[0] for c in caps):
        return list(tensors), caps[0]
    return [t.contiguous() for t in tensors], n_rows


def quantize(x, group_size: int = 64, bits: int = 8):
    """Affine 8-bit quantisation over the last axis (the role of ``mx.quantize`` on the cache write path).

    Returns ``(wq uint32 [..., D/4], scales [..., D/64], biases [..., D/64])``; scales and biases in
    the dtype of ``x``.
    """
    if group_size != 64 or bits != 8:
        raise ValueError("quantize supports group_size=64, bits=8 only")
    if x.dtype not in _lib.DTYPE_CODE:
        raise ValueError("x must be float32, float16 or bfloat16")
    if x.ndim < 1 or int(x.shape[-1]) % 64 != 0 or x.numel() == 0:
        raise ValueError("the last axis must be a non-empty multiple of the group size 64")
    dev = _lib.require_device(x)
    xc = x.contiguous()
    d = int(xc.shape[-1])
    lead = tuple(xc.shape[:-1])
    wq = torch.empty(lead + (d // 4,), dtype=torch.int32, device=dev).view(torch.uint32)
    scales = torch.empty(lead + (d // 64,), dtype=xc.dtype, device=dev)
    biases = torch.empty_like(scales)
    _lib.check(_lib.lib().mspr_affine_q8_quantize(
        _lib.ptr(xc), _lib.DTYPE_CODE[xc.dtype], xc.numel() // 64, _lib.ptr(wq), _lib.ptr(scales), _lib.ptr(biases),
        64, 8, _lib.stream_ptr()), "quantize")
    return wq, scales, biases


def dequantize(wq, scales, biases, group_size: int = 64, bits: int = 8):
    """``code * scale + bias`` in the dtype of ``scales`` (the role of ``mx.dequantize``)."""
    if group_size != 64 or bits != 8:
        raise ValueError("dequantize supports group_size=64, bits=8 only")
    if scales.dtype not in _lib.DTYPE_CODE or biases.dtype != scales.dtype:
        raise ValueError("scales and biases must share a float32/float16/bfloat16 dtype")
    if wq.dtype not in (torch.uint32, torch.int32):
        raise ValueError("codes must be uint32 words")
    if tuple(scales.shape) != tuple(biases.shape) or tuple(wq.shape[:-1]) != tuple(scales.shape[:-1]) or \
            int(wq.shape[-1]) != 16 * int(scales.shape[-1]) or wq.numel() == 0:
        raise ValueError("codes, scales and biases disagree on the group layout")
    dev = _lib.require_device(wq, scales, biases)
    w, s, b = wq.contiguous(), scales.contiguous(), biases.contiguous()
    out = torch.empty(tuple(w.shape[:-1]) + (int(w.shape[-1]) * 4,), dtype=s.dtype, device=dev)
    _lib.check(_lib.lib().mspr_affine_q8_dequantize(
        _lib.ptr(w), _lib.ptr(s), _lib.ptr(b), _lib.DTYPE_CODE[s.dtype], s.numel(), _lib.ptr(out), 64, 8,
        _lib.stream_ptr()), "dequantize")
    return out


class QuantizedKVCache:
    """Affine 8-bit KV cache with quantise-on-append (the role of mlx_lm's ``QuantizedKVCache`` in
    runtime/qwen/full_attention.py:315,352-356).

    ``keys`` / ``values`` are ``(wq, scales, biases)`` triplets over a capacity that grows in
    ``step``-token blocks; ``offset`` tokens are valid. ``update_and_fetch`` quantises the new rows in
    place behind the valid prefix and returns the triplets trimmed to the new length; ``state`` is the
    same view without an update.
    """

    step = 256

    def __init__(self, group_size: int = 64, bits: int = 8):
        if group_size != 64 or bits != 8:
            raise ValueError("QuantizedKVCache supports group_size=64, bits=8 only")
        self.group_size = group_size
        self.bits = bits
        self.offset = 0
        self.keys = None
        self.values = None

    def _grow(self, like, need: int):
        B, H, _, D = (int(v) for v in like.shape)
        cap = 0 if self.keys is None else int(self.keys[0].shape[2])
        if need <= cap:
            return
        new_cap = (need + self.step - 1) // self.step * self.step

        def alloc():
            return (torch.zeros((B, H, new_cap, D // 4), dtype=torch.int32, device=like.device).view(torch.uint32),
                    torch.zeros((B, H, new_cap, D // 64), dtype=like.dtype, device=like.device),
                    torch.zeros((B, H, new_cap, D // 64), dtype=like.dtype, device=like.device))

        new_k, new_v = alloc(), alloc()
        if self.keys is not None and self.offset:
            for old, new in zip(self.keys + self.values, new_k + new_v):
                new[:, :, :self.offset].view(torch.int32 if new.dtype == torch.uint32 else new.dtype).copy_(
                    old[:, :, :self.offset].view(torch.int32 if old.dtype == torch.uint32 else old.dtype))
        self.keys, self.values = new_k, new_v

    def _trimmed(self, triplet):
        return tuple(t[:, :, :self.offset] for t in triplet)

    @property
    def state(self):
        if self.keys is None:
            return None, None
        return self._trimmed(self.keys), self._trimmed(self.values)

    def update_and_fetch(self, keys, values):
        """Append ``keys``/``values`` ``[B, Hkv, L, D]`` and return the quantised cache up to the new length."""
        if keys.ndim != 4 or tuple(keys.shape) != tuple(values.shape):
            raise ValueError("keys and values must be [B, Hkv, L, D] of one shape")
        L = int(keys.shape[2])
        self._grow(keys, self.offset + L)
        for src, dst in ((keys, self.keys), (values, self.values)):
            wq, sc, bi = quantize(src)
            lo, hi = self.offset, self.offset + L
            dst[0][:, :, lo:hi].view(torch.int32).copy_(wq.view(torch.int32))
            dst[1][:, :, lo:hi].copy_(sc)
            dst[2][:, :, lo:hi].copy_(bi)
        self.offset += L
        return self._trimmed(self.keys), self._trimmed(self.values)


def sdpa_decode_q8(queries, k_wq, k_scales, k_biases, v_wq, v_scales, v_biases, scale, *, group_size: int = 64,
                   bits: int = 8, workspace=None, **_tuning):
    """One-token GQA attention over an affine 8-bit KV cache (reference call site full_attention.py:323).

    Args:
        queries: float32 ``[B, Hq, 1, 256]`` (already rotated).
        k_wq, k_scales, k_biases / v_wq, v_scales, v_biases: the quantised cache of ``N`` tokens.
        scale: softmax scale.

    Returns:
        float32 ``[B, Hq, 1, 256]``.
    """
    if group_size != 64 or bits != 8:
        raise ValueError("sdpa_decode_q8 supports group_size=64, bits=8 only")
    if queries.ndim != 4 or int(queries.shape[2]) != 1:
        raise ValueError("queries must be [B, Hq, 1, D] (single-token decode)")
    if int(queries.shape[3]) != _HEAD_DIM:
        raise ValueError("q8 attention requires head_dim=256")
    if queries.dtype != torch.float32:
        raise ValueError("queries must be float32")
    B, Hq = int(queries.shape[0]), int(queries.shape[1])
    _check_q8_triplet("key", k_wq, k_scales, k_biases, B)
    N = int(k_wq.shape[2])
    _check_q8_triplet("value", v_wq, v_scales, v_biases, B, N)
    Hkv = int(k_wq.shape[1])
    if int(v_wq.shape[1]) != Hkv or Hq % Hkv != 0 or Hq // Hkv > 16:
        raise ValueError("query heads must be a multiple (at most 16x) of the KV heads")
    if k_scales.dtype != v_scales.dtype:
        raise ValueError("key and value scales must share a dtype")
    if N < 1:
        raise ValueError("the cache must hold at least one token")
    _lib.require_device(queries, k_wq, k_scales, k_biases, v_wq, v_scales, v_biases)
    q = queries.contiguous()
    (kw, ks, kb, vw, vs, vb), kv_rows = _cache_operands((k_wq, k_scales, k_biases, v_wq, v_scales, v_biases), N)
    out = torch.empty_like(q)
    if workspace is None:
        workspace = _lib.q8_decode_workspace(B, Hkv, N, q.device)
    _lib.check(_lib.lib().mspr_sdpa_decode_q8(
        _lib.ptr(q), _lib.DTYPE_CODE[q.dtype], _lib.ptr(kw), _lib.ptr(ks), _lib.ptr(kb), _lib.ptr(vw), _lib.ptr(vs),
        _lib.ptr(vb), _lib.DTYPE_CODE[ks.dtype], B, Hq, Hkv, _HEAD_DIM, N, kv_rows, float(scale), 64, 8, _lib.ptr(out),
        _lib.ptr(workspace), workspace.numel() * workspace.element_size(), _lib.stream_ptr()), "sdpa_decode_q8")
    return out


def sdpa_decode_q8_0(queries, k_codes, k_scales, v_codes, v_scales, scale, *, workspace=None):
    """One-token GQA attention over a Q8_0 KV cache (int8 codes, one float16 scale per 32 elements).

    Args:
        queries: ``[B, Hq, 256]`` float32, float16 or bfloat16.
        k_codes, v_codes: int8 ``[B, Hkv, N, 256]``; k_scales, v_scales: float16 ``[B, Hkv, N, 8]``.

    Returns:
        ``[B, Hq, 256]`` in the dtype of ``queries``.
    """
    if queries.ndim != 3 or int(queries.shape[2]) != _HEAD_DIM:
        raise ValueError("queries must be [B, Hq, 256]")
    if queries.dtype not in _lib.DTYPE_CODE:
        raise ValueError("queries must be float32, float16 or bfloat16")
    B, Hq = int(queries.shape[0]), int(queries.shape[1])
    for name, c, s in (("key", k_codes, k_scales), ("value", v_codes, v_scales)):
        if c.ndim != 4 or c.dtype != torch.int8 or int(c.shape[3]) != _HEAD_DIM:
            raise ValueError(f"{name} codes must be int8 [B, Hkv, N, 256]")
        if s.dtype != torch.float16 or tuple(s.shape) != tuple(c.shape[:3]) + (_HEAD_DIM // 32,):
            raise ValueError(f"{name} scales must be float16 [B, Hkv, N, 8]")
        if int(c.shape[0]) != B:
            raise ValueError(f"{name} cache batch must match queries")
    if tuple(k_codes.shape) != tuple(v_codes.shape):
        raise ValueError("keys and values disagree on the number of cached tokens")
    Hkv, N = int(k_codes.shape[1]), int(k_codes.shape[2])
    if Hq % Hkv != 0 or Hq // Hkv > 16:
        raise ValueError("query heads must be a multiple (at most 16x) of the KV heads")
    if N < 1:
        raise ValueError("the cache must hold at least one token")
    _lib.require_device(queries, k_codes, k_scales, v_codes, v_scales)
    q = queries.contiguous()
    (kc, ks, vc, vs), kv_rows = _cache_operands((k_codes, k_scales, v_codes, v_scales), N)
    out = torch.empty_like(q)
    if workspace is None:
        workspace = _lib.q8_decode_workspace(B, Hkv, N, q.device)
    _lib.check(_lib.lib().mspr_sdpa_decode_q8_0(
        _lib.ptr(q), _lib.DTYPE_CODE[q.dtype], _lib.ptr(kc), _lib.ptr(ks), _lib.ptr(vc), _lib.ptr(vs), B, Hq, Hkv,
        _HEAD_DIM, N, kv_rows, float(scale), _lib.ptr(out), _lib.ptr(workspace),
        workspace.numel() * workspace.element_size(), _lib.stream_ptr()), "sdpa_decode_q8_0")
    return out


def sdpa_fa_prefill_q8(queries, pk_wq, pk_scales, pk_biases, pv_wq, pv_scales, pv_biases, self_k, self_v, scale, *,
                       group_size: int = 64, bits: int = 8, workspace=None, **_tuning):
    """Causal flash prefill over a quantised prefix plus the dense chunk (reference call site full_attention.py:372).

    Args:
        queries: float32 ``[B, Hq, L, 256]`` (already rotated).
        pk_* / pv_*: the affine 8-bit prefix of ``P`` tokens as read from the cache *before* the chunk
            was appended (``P`` may be 0).
        self_k, self_v: ``[B, Hkv, L, 256]`` float32/float16/bfloat16, the chunk's own keys and values
            after the 8-bit round trip.
        scale: softmax scale.

    Returns:
        float32 ``[B, Hq, L, 256]``; row ``i`` attends all prefix keys and chunk keys ``[0, i]``.
    """
    if group_size != 64 or bits != 8:
        raise ValueError("sdpa_fa_prefill_q8 supports group_size=64, bits=8 only")
    if queries.ndim != 4 or int(queries.shape[3]) != _HEAD_DIM:
        raise ValueError("queries must be [B, Hq, L, 256]")
    if queries.dtype != torch.float32:
        raise ValueError("queries must be float32")
    B, Hq, L = int(queries.shape[0]), int(queries.shape[1]), int(queries.shape[2])
    _check_q8_triplet("past key", pk_wq, pk_scales, pk_biases, B)
    P = int(pk_wq.shape[2])
    _check_q8_triplet("past value", pv_wq, pv_scales, pv_biases, B, P)
    Hkv = int(pk_wq.shape[1])
    if pk_scales.dtype != pv_scales.dtype:
        raise ValueError("key and value scales must share a dtype")
    if self_k.ndim != 4 or tuple(self_k.shape) != (B, Hkv, L, _HEAD_DIM) or tuple(self_v.shape) != tuple(self_k.shape):
        raise ValueError("self_k and self_v must be [B, Hkv, L, 256] with the chunk length of queries")
    if self_k.dtype != self_v.dtype or self_k.dtype not in _lib.DTYPE_CODE:
        raise ValueError("self_k and self_v must share a float32/float16/bfloat16 dtype")
    if Hq % Hkv != 0 or Hq // Hkv not in (1, 2, 4, 8):
        raise ValueError("query heads per KV head must be 1, 2, 4 or 8")
    if L < 1:
        raise ValueError("the chunk must hold at least one token")
    _lib.require_device(queries, pk_wq, pk_scales, pk_biases, pv_wq, pv_scales, pv_biases, self_k, self_v)
    q, sk, sv = queries.contiguous(), self_k.contiguous(), self_v.contiguous()
    (kw, ks, kb, vw, vs, vb), past_rows = _cache_operands(
        (pk_wq, pk_scales, pk_biases, pv_wq, pv_scales, pv_biases), P)
    out = torch.empty_like(q)
    if workspace is None:
        nbytes = int(_lib.lib().mspr_sdpa_fa_prefill_q8_workspace_bytes(B, Hq, Hkv, L, P))
        workspace = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=q.device)
    _lib.check(_lib.lib().mspr_sdpa_fa_prefill_q8(
        _lib.ptr(q), _lib.ptr(kw), _lib.ptr(ks), _lib.ptr(kb), _lib.ptr(vw), _lib.ptr(vs), _lib.ptr(vb),
        _lib.DTYPE_CODE[ks.dtype], _lib.ptr(sk), _lib.ptr(sv), _lib.DTYPE_CODE[sk.dtype], B, Hq, Hkv, _HEAD_DIM, L, P,
        past_rows, float(scale), 64, 8, _lib.ptr(out), _lib.ptr(workspace), workspace.numel() * workspace.element_size(),
        _lib.stream_ptr()), "sdpa_fa_prefill_q8")
    return out


def flash_prefill(queries, keys, values, scale, *, past_len: int, workspace=None):
    """Causal chunked-prefill GQA attention over a dense 16-bit cache that already holds the chunk.

    Query row ``i`` sits at position ``past_len + i`` and attends keys ``[0, past_len + i]``: the
    arithmetic of the reference's composed prefill route (``scaled_dot_product_attention`` with
    ``mask="causal"`` over the fetched cache, full_attention.py:399-409).

    Args:
        queries: ``[B, Hq, L, 256]`` float16 or bfloat16.
        keys, values: ``[B, Hkv, rows, 256]`` of the same dtype, ``rows >= past_len + L``.

    Returns:
        ``[B, Hq, L, 256]`` in the dtype of ``queries``.
    """
    if queries.ndim != 4 or keys.ndim != 4 or values.ndim != 4:
        raise ValueError("queries, keys and values must be rank-4 [B, H, T, D]")
    if int(queries.shape[3]) != _HEAD_DIM or int(keys.shape[3]) != _HEAD_DIM or int(values.shape[3]) != _HEAD_DIM:
        raise ValueError("flash prefill requires head_dim=256")
    if queries.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("queries must be float16 or bfloat16")
    if keys.dtype != queries.dtype or values.dtype != queries.dtype:
        raise ValueError("keys and values must have the dtype of queries")
    if tuple(keys.shape) != tuple(values.shape) or int(keys.shape[0]) != int(queries.shape[0]):
        raise ValueError("keys and values must share a shape and the batch of queries")
    B, Hq, L = int(queries.shape[0]), int(queries.shape[1]), int(queries.shape[2])
    Hkv, rows = int(keys.shape[1]), int(keys.shape[2])
    if Hq % Hkv != 0 or Hq // Hkv not in (1, 2, 4, 8):
        raise ValueError("query heads per KV head must be 1, 2, 4 or 8")
    past_len = int(past_len)
    if L < 1 or past_len < 0 or past_len + L > rows:
        raise ValueError("need q_len >= 1, past_len >= 0 and past_len + q_len <= cache rows")
    _lib.require_device(queries, keys, values)
    q, k, v = queries.contiguous(), keys.contiguous(), values.contiguous()
    out = torch.empty_like(q)
    if workspace is None:
        nbytes = int(_lib.lib().mspr_flash_prefill_workspace_bytes(B, Hq, Hkv, L, past_len))
        workspace = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=q.device)
    _lib.check(_lib.lib().mspr_flash_prefill(
        _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.DTYPE_CODE[q.dtype], B, Hq, Hkv, _HEAD_DIM, L, past_len, rows,
        float(scale), _lib.ptr(out), _lib.ptr(workspace), workspace.numel() * workspace.element_size(),
        _lib.stream_ptr()), "flash_prefill")
    return out
