"""DS4 decode indexer pre-top-k operators on MI355X.

Mirror of the reference module
``src/moespresso/runtime/deepseek_v4/indexer_score_kernel.py``: the same
callables, argument meaning and rejections, on ``torch.Tensor`` operands that
live on a HIP device. Every callable validates shapes and dtypes first (so a
rejection is a ``ValueError`` whatever device the tensors are on) and then
launches a hand-written gfx950 kernel through the C-ABI; there is no composed
or CPU fallback.

Numerical contract of the QAT (reference ``indexer_score_kernel.py:13-34``):
radix-2 Hadamard butterflies in increasing stride order in float32, the
``exp(ceil(log(amax/6)/ln2)*ln2)`` group scale with float32 steps, first-wins
nearest lattice value, NaN-passthrough clip. The log and exp of the scale are
correctly rounded float32 here.
"""

from __future__ import annotations

import math
import os

import torch

from moespresso_amd import _lib

# Gate for the fused decode pre-top-k path (reference indexer_score_kernel.py:63):
# the wrapper layers consult it, the kernels below run regardless.
_ENABLED = False

_HEAD_DIM = 128
_MAX_HEADS = 64

_HADAMARD_SCALE = 0.08838834764831845
_AMAX_FLOOR = 7.052966104933725e-38
_LN2 = math.log(2.0)

_CHAIN_TRIMS_ENV = "MOESPRESSO_DSV4_INDEXER_CHAIN_TRIMS"
_SCORE_TAIL_ENV = "MOESPRESSO_DSV4_INDEXER_SCORE_TAIL"

_TAIL_MIN_HEADS = 32
_TAIL_MAX_HEADS = 64


def _metal_available() -> bool:
    """Name kept from the reference (:235); reports HIP device + kernel library."""
    return _lib.hip_available()


def _query_dtypes():
    return (torch.float32, torch.float16, torch.bfloat16)


def indexer_qat_rows(x: torch.Tensor) -> torch.Tensor:
    """DS4 indexer QAT over 128-wide rows (reference ``indexer_qat_rows``, :284).

    Args:
        x: ``[..., 128]`` float32, float16 or bfloat16 rows.

    Returns:
        float32 tensor of the same shape.
    """
    if x.ndim < 1 or int(x.shape[-1]) != _HEAD_DIM:
        raise ValueError("indexer QAT expects 128-wide rows")
    if x.dtype not in _query_dtypes():
        raise ValueError("indexer QAT rows must be float32, float16, or bfloat16")
    n_rows = x.numel() // _HEAD_DIM
    if n_rows == 0:
        raise ValueError("indexer QAT expects at least one row")
    _lib.require_device(x)
    rows2d = x.reshape(-1, _HEAD_DIM).contiguous()
    out = torch.empty((n_rows, _HEAD_DIM), dtype=torch.float32, device=x.device)
    rc = _lib.lib().mspr_indexer_qat_rows(
        _lib.ptr(rows2d), _lib.DTYPE_CODE[x.dtype], n_rows, _lib.ptr(out), _lib.stream_ptr())
    _lib.check(rc, "indexer_qat_rows")
    return out.reshape(x.shape)


def fused_qat_scores_eligible(q, pooled_qat, weights) -> bool:
    """Shape/dtype predicate of the fused decode score row (reference :321)."""
    if not _ENABLED or not _metal_available():
        return False
    if q.ndim != 4 or pooled_qat.ndim != 3 or weights.ndim != 3:
        return False
    batch, n_heads, tokens, head_dim = (int(v) for v in q.shape)
    if batch != 1 or tokens != 1 or head_dim != _HEAD_DIM:
        return False
    if n_heads <= 0 or n_heads > _MAX_HEADS:
        return False
    if int(pooled_qat.shape[0]) != 1 or int(pooled_qat.shape[2]) != head_dim:
        return False
    if int(pooled_qat.shape[1]) <= 0:
        return False
    if tuple(int(v) for v in weights.shape) != (1, 1, n_heads):
        return False
    if q.dtype not in _query_dtypes():
        return False
    if pooled_qat.dtype != torch.float32 or weights.dtype != torch.float32:
        return False
    return True


def fused_qat_indexer_scores(q, pooled_qat, weights, scale) -> torch.Tensor:
    """Decode indexer score row with the query QAT in-kernel (reference :354).

    Args:
        q: ``[1, n_heads, 1, 128]`` post-rope, pre-QAT queries (f32/f16/bf16).
        pooled_qat: float32 ``[1, n_rows, 128]`` QAT'd pool rows.
        weights: float32 ``[1, 1, n_heads]`` head weights (already ``* n_heads**-0.5``).
        scale: per-head score scale (``head_dim ** -0.5``).

    Returns:
        float32 ``[n_rows]``:
        ``scores[r] = sum_h max(qat(q_h) . pooled_r, 0) * scale * weights[h]``.
    """
    if q.ndim != 4:
        raise ValueError("q must have shape [1, n_heads, 1, 128]")
    batch, n_heads, tokens, head_dim = (int(v) for v in q.shape)
    if batch != 1 or tokens != 1:
        raise ValueError("fused indexer scoring handles one decode token")
    if head_dim != _HEAD_DIM:
        raise ValueError("DS4 fused indexer scoring requires head_dim=128")
    if n_heads <= 0 or n_heads > _MAX_HEADS:
        raise ValueError("q must carry between 1 and 64 heads")
    if pooled_qat.ndim != 3 or int(pooled_qat.shape[0]) != 1 or int(pooled_qat.shape[2]) != head_dim:
        raise ValueError("pooled_qat must have shape [1, n_rows, 128]")
    n_rows = int(pooled_qat.shape[1])
    if n_rows <= 0:
        raise ValueError("pooled_qat must contain at least one row")
    if tuple(int(v) for v in weights.shape) != (1, 1, n_heads):
        raise ValueError("weights must have shape [1, 1, n_heads]")
    if q.dtype not in _query_dtypes():
        raise ValueError("q must be float32, float16, or bfloat16")
    if pooled_qat.dtype != torch.float32 or weights.dtype != torch.float32:
        raise ValueError("pooled_qat and weights must be float32")
    _lib.require_device(q, pooled_qat, weights)
    qc = q.reshape(n_heads, head_dim).contiguous()
    pc = pooled_qat.reshape(n_rows, head_dim).contiguous()
    wc = weights.reshape(n_heads).contiguous()
    scores = torch.empty((n_rows,), dtype=torch.float32, device=q.device)
    rc = _lib.lib().mspr_fused_qat_indexer_scores(
        _lib.ptr(qc), _lib.DTYPE_CODE[q.dtype], n_heads, _lib.ptr(pc), n_rows, _lib.ptr(wc),
        float(scale), _lib.ptr(scores), _lib.stream_ptr())
    _lib.check(rc, "fused_qat_indexer_scores")
    return scores


def score_tail_enabled() -> bool:
    """Env kill switches read per call (reference :499)."""
    if os.environ.get(_CHAIN_TRIMS_ENV, "1") == "0":
        return False
    if os.environ.get(_SCORE_TAIL_ENV, "1") == "0":
        return False
    return _metal_available()


def score_tail_eligible(scores, weights_raw, params) -> bool:
    """Shape/dtype predicate of the fused score tail (reference :530)."""
    if not score_tail_enabled():
        return False
    if scores.ndim != 4 or weights_raw.ndim != 3:
        return False
    batch, n_heads, tokens, capacity = (int(v) for v in scores.shape)
    if batch != 1 or tokens != 1 or capacity <= 0:
        return False
    if not _TAIL_MIN_HEADS <= n_heads <= _TAIL_MAX_HEADS:
        return False
    if scores.dtype != torch.float32:
        return False
    if tuple(int(v) for v in weights_raw.shape) != (1, 1, n_heads):
        return False
    if weights_raw.dtype not in _query_dtypes():
        return False
    if params.dtype != torch.int32 or params.numel() < 2:
        return False
    return True


def fused_score_tail(scores, weights_raw, params, *, scale) -> torch.Tensor:
    """Finish the fixed-state score chain in one launch (reference :562).

    Args:
        scores: float32 ``[1, n_heads, 1, capacity]`` score matmul output.
        weights_raw: ``[1, 1, n_heads]`` raw head-weight projection (f32/f16/bf16).
        params: int32 array whose second element is the valid pool row count.
        scale: per-head score scale.

    Returns:
        float32 ``[1, 1, capacity]``: ``-sum_h relu(s)*scale*(w*n_heads**-0.5)`` on
        the valid prefix and ``+inf`` on the tail. Each step rounds to float32;
        lane ``l`` of a 32-lane group adds heads ``l, l+32`` and the partials are
        combined by an xor butterfly (offsets 16, 8, 4, 2, 1).
    """
    if scores.ndim != 4:
        raise ValueError("scores must have shape [1, n_heads, 1, capacity]")
    batch, n_heads, tokens, capacity = (int(v) for v in scores.shape)
    if batch != 1 or tokens != 1:
        raise ValueError("the fused score tail handles one decode token")
    if capacity <= 0:
        raise ValueError("scores must cover at least one capacity column")
    if not _TAIL_MIN_HEADS <= n_heads <= _TAIL_MAX_HEADS:
        raise ValueError("the score tail transcription covers 32 to 64 index heads")
    if scores.dtype != torch.float32:
        raise ValueError("scores must be float32")
    if tuple(int(v) for v in weights_raw.shape) != (1, 1, n_heads):
        raise ValueError("weights_raw must have shape [1, 1, n_heads]")
    if weights_raw.dtype not in _query_dtypes():
        raise ValueError("weights_raw must be float32, float16, or bfloat16")
    if params.dtype != torch.int32 or params.numel() < 2:
        raise ValueError("params must be int32 with the row count at index 1")
    _lib.require_device(scores, weights_raw, params)
    sc = scores.reshape(n_heads, capacity).contiguous()
    wc = weights_raw.reshape(n_heads).contiguous()
    pc = params.reshape(-1).contiguous()
    neg = torch.empty((capacity,), dtype=torch.float32, device=scores.device)
    rc = _lib.lib().mspr_indexer_score_tail(
        _lib.ptr(sc), n_heads, capacity, _lib.ptr(wc), _lib.DTYPE_CODE[weights_raw.dtype],
        _lib.ptr(pc), float(scale), _lib.ptr(neg), _lib.stream_ptr())
    _lib.check(rc, "fused_score_tail")
    return neg.reshape(1, 1, capacity)


# ----------------------------------------------------------------------------
# Extensions beyond the reference module (BASELINE config 4 shapes).
# ----------------------------------------------------------------------------

def topk_select(scores: torch.Tensor, topk: int) -> torch.Tensor:
    """Deterministic top-k of float32 score rows.

    Stands in for ``mx.argpartition(-scores, kth=k-1)[..., :k]`` (reference
    ``model.py:1003``) with a defined order: rows strictly above the k-th value
    in ascending row order, then the lowest-index rows tied with it (the
    emission order of the reference prep kernel, ``decode_attention_kernel.py:
    337-375``).

    Args:
        scores: float32 ``[..., n_rows]``; the selection runs over the last axis.
        topk: ``0 < topk <= n_rows``.

    Returns:
        int32 ``[..., topk]``.
    """
    if scores.ndim < 1:
        raise ValueError("scores must have a row axis")
    if scores.dtype != torch.float32:
        raise ValueError("scores must be float32")
    n_rows = int(scores.shape[-1])
    topk = int(topk)
    if not 0 < topk <= n_rows:
        raise ValueError("topk must be positive and at most n_rows")
    _lib.require_device(scores)
    s2 = scores.reshape(-1, n_rows).contiguous()
    batch = int(s2.shape[0])
    sel = torch.empty((batch, topk), dtype=torch.int32, device=scores.device)
    rc = _lib.lib().mspr_topk_select(_lib.ptr(s2), n_rows, batch, n_rows, topk, _lib.ptr(sel),
                                     _lib.stream_ptr())
    _lib.check(rc, "topk_select")
    return sel.reshape(*scores.shape[:-1], topk)


def indexer_scores_fp8(q, keys, key_scales, weights) -> torch.Tensor:
    """Batched lightning-indexer score rows with FP8 keys (BASELINE config 4 shape).

    ``scores[b, r] = sum_h weights[b, h] * relu(q[b, h] . e4m3(keys[b, r])) * key_scales[b, r]``.
    The batched, fp8-key extension of ``fused_qat_indexer_scores`` (whose
    reference form takes float32 pool rows, batch 1, and QATs the query).

    Args:
        q: bfloat16 ``[batch, n_heads, 128]``, ``n_heads <= 64``.
        keys: E4M3FN ``[batch, n_rows, 128]`` (``torch.float8_e4m3fn`` or ``uint8`` bytes).
        key_scales: float32 ``[batch, n_rows]`` positive per-key scales.
        weights: float32 ``[batch, n_heads]`` head weights.

    Returns:
        float32 ``[batch, n_rows]``.
    """
    if q.ndim != 3 or int(q.shape[2]) != _HEAD_DIM:
        raise ValueError("q must have shape [batch, n_heads, 128]")
    batch, n_heads, _ = (int(v) for v in q.shape)
    if n_heads <= 0 or n_heads > _MAX_HEADS:
        raise ValueError("q must carry between 1 and 64 heads")
    if q.dtype != torch.bfloat16:
        raise ValueError("q must be bfloat16")
    if keys.ndim != 3 or int(keys.shape[0]) != batch or int(keys.shape[2]) != _HEAD_DIM:
        raise ValueError("keys must have shape [batch, n_rows, 128]")
    if keys.dtype not in (torch.float8_e4m3fn, torch.uint8):
        raise ValueError("keys must be float8_e4m3fn (or its uint8 bytes)")
    n_rows = int(keys.shape[1])
    if n_rows <= 0:
        raise ValueError("keys must contain at least one row")
    if tuple(int(v) for v in key_scales.shape) != (batch, n_rows) or key_scales.dtype != torch.float32:
        raise ValueError("key_scales must be float32 [batch, n_rows]")
    if tuple(int(v) for v in weights.shape) != (batch, n_heads) or weights.dtype != torch.float32:
        raise ValueError("weights must be float32 [batch, n_heads]")
    dev = _lib.require_device(q, keys, key_scales, weights)
    qc, kc, sc, wc = q.contiguous(), keys.contiguous(), key_scales.contiguous(), weights.contiguous()
    scores = torch.empty((batch, n_rows), dtype=torch.float32, device=dev)
    rc = _lib.lib().mspr_indexer_scores_fp8(_lib.ptr(qc), _lib.ptr(kc), _lib.ptr(sc), _lib.ptr(wc), batch,
                                            n_heads, n_rows, _lib.ptr(scores), _lib.stream_ptr())
    _lib.check(rc, "indexer_scores_fp8")
    return scores
