"""Fused DS4 ratio-4 decode attention island on MI355X.

Mirror of the reference module
``src/moespresso/runtime/deepseek_v4/decode_attention_kernel.py``:

- ``fused_decode_prep``: indexer query QAT (staged as float16), score row,
  deterministic radix top-k, prepared KV row (rope tail + E4M3FN prefix);
- ``fused_decode_sdpa``: rope(q), online-softmax attention over the local
  window (prepared row substituted at the write slot) plus the selected pool
  rows, per-head sink, float16 output, inverse rope;
- ``fp8_kv_prefix_rows``: standalone E4M3FN round trip of 512-wide rows.

The reference runs the prep inside one 1024-thread threadgroup and the SDPA
with one threadgroup per head; here the score row and the attention are spread
over the whole device (split over pool rows, merged by log-sum-exp). Operands
are ``torch.Tensor`` on a HIP device; validation errors are ``ValueError`` with
the reference's wording.
"""

from __future__ import annotations

import math

import torch

from moespresso_amd import _lib
from moespresso_amd.runtime.deepseek_v4.indexer_score_kernel import _metal_available

# Gate of the fused island (reference decode_attention_kernel.py:86); wrapper
# layers consult it, the kernels run regardless.
_ENABLED = False

_HEAD_DIM = 512
_ROPE_DIM = 64
_INDEX_HEAD_DIM = 128
_MAX_HEADS = 64

_LN2 = math.log(2.0)


def _query_dtypes():
    return (torch.float32, torch.float16, torch.bfloat16)


def fp8_kv_prefix_rows(x: torch.Tensor) -> torch.Tensor:
    """E4M3FN round trip of dims [0, 448) of 512-wide float32 rows (reference :587).

    Per 64-element block: ``amax = max(|x|, 1e-4)``, power-of-two scale
    ``exp(ceil(log(amax/448)/ln2)*ln2)``, clip to +-448, nearest of the 127
    non-negative E4M3FN values with exact ties to the lower value. Dims
    [448, 512) are copied.
    """
    if x.ndim < 1 or int(x.shape[-1]) != _HEAD_DIM:
        raise ValueError("fp8 rows expect 512-wide rows")
    if x.dtype != torch.float32:
        raise ValueError("fp8 rows must be float32")
    n_rows = x.numel() // _HEAD_DIM
    if n_rows == 0:
        raise ValueError("fp8 rows expect at least one row")
    _lib.require_device(x)
    rows2d = x.reshape(-1, _HEAD_DIM).contiguous()
    out = torch.empty_like(rows2d)
    rc = _lib.lib().mspr_fp8_kv_prefix_rows(_lib.ptr(rows2d), n_rows, _lib.ptr(out), _lib.stream_ptr())
    _lib.check(rc, "fp8_kv_prefix_rows")
    return out.reshape(x.shape)


def fused_decode_prep(q_idx, pooled_qat, weights, kv_row, inv_freq, params, *, scale, topk,
                      pool_rows_in_params: bool = False):
    """Score, select, and prepare the KV row for one ratio-4 decode token (reference :669).

    With ``pool_rows_in_params`` (an extension for the fixed-capacity decode state, reference
    fixed_decode_state.py:186-206) ``pooled_qat`` is a capacity buffer and ``params`` is int32
    ``[position, write_idx, rows in use]``: the row count is read on the device, rows not in use score
    ``-inf``, so a launch captured in a HIP graph follows the pool as it grows.

    Args:
        q_idx: ``[n_heads, 128]`` post-rope, pre-QAT indexer queries (f32/f16/bf16).
        pooled_qat: float32 ``[n_rows, 128]`` QAT'd indexer pool rows.
        weights: float32 ``[n_heads]`` head weights (already ``* n_heads**-0.5``).
        kv_row: float16 ``[512]`` post-norm, pre-rope KV projection row.
        inv_freq: float32 ``[32]`` rope inverse frequencies (YaRN folded).
        params: int32 array whose first element is the token position.
        scale: indexer score scale (``index_head_dim ** -0.5``).
        topk: selection width; must be smaller than ``n_rows``.

    Returns:
        ``(sel, row, scores)``: int32 ``[topk]`` (rows above the k-th score in
        ascending row order, then boundary ties by ascending row), float16
        ``[512]`` roped + FP8-rounded KV row, float32 ``[n_rows]`` scores.
    """
    if q_idx.ndim != 2 or int(q_idx.shape[1]) != _INDEX_HEAD_DIM:
        raise ValueError("q_idx must have shape [n_heads, 128]")
    n_heads = int(q_idx.shape[0])
    if n_heads <= 0 or n_heads > _MAX_HEADS:
        raise ValueError("q_idx must carry between 1 and 64 heads")
    if q_idx.dtype not in _query_dtypes():
        raise ValueError("q_idx must be float32, float16, or bfloat16")
    if (pooled_qat.ndim != 2 or int(pooled_qat.shape[1]) != _INDEX_HEAD_DIM
            or pooled_qat.dtype != torch.float32):
        raise ValueError("pooled_qat must be float32 [n_rows, 128]")
    n_rows = int(pooled_qat.shape[0])
    topk = int(topk)
    if not 0 < topk < n_rows:
        raise ValueError("topk must be positive and smaller than n_rows")
    # The reference also rejects n_rows >= 65536 ("the radix-select scan packs
    # counts in 16 bits"); the scan here uses 32-bit counters, so longer pools
    # are accepted.
    if tuple(int(v) for v in weights.shape) != (n_heads,) or weights.dtype != torch.float32:
        raise ValueError("weights must be float32 [n_heads]")
    if tuple(int(v) for v in kv_row.shape) != (_HEAD_DIM,) or kv_row.dtype != torch.float16:
        raise ValueError("kv_row must be float16 [512]")
    if int(inv_freq.shape[-1]) != _ROPE_DIM // 2 or inv_freq.dtype != torch.float32:
        raise ValueError("inv_freq must be float32 [32]")
    if params.dtype != torch.int32 or params.numel() < 1:
        raise ValueError("params must be int32 with the position at index 0")
    if pool_rows_in_params and params.numel() < 3:
        raise ValueError("params must be int32 [position, write_idx, pool_rows] for a fixed-capacity pool")
    dev = _lib.require_device(q_idx, pooled_qat, weights, kv_row, inv_freq, params)
    qc = q_idx.contiguous()
    pc = pooled_qat.contiguous()
    wc = weights.contiguous()
    kc = kv_row.contiguous()
    fc = inv_freq.reshape(-1).contiguous()
    prm = params.reshape(-1).contiguous()
    sel = torch.empty((topk,), dtype=torch.int32, device=dev)
    row = torch.empty((_HEAD_DIM,), dtype=torch.float16, device=dev)
    scores = torch.empty((n_rows,), dtype=torch.float32, device=dev)
    entry = _lib.lib().mspr_fused_decode_prep_fixed if pool_rows_in_params else _lib.lib().mspr_fused_decode_prep
    rc = entry(
        _lib.ptr(qc), _lib.DTYPE_CODE[q_idx.dtype], n_heads, _lib.ptr(pc), n_rows, _lib.ptr(wc),
        _lib.ptr(kc), _lib.ptr(fc), _lib.ptr(prm), float(scale), topk, _lib.ptr(sel), _lib.ptr(row),
        _lib.ptr(scores), _lib.stream_ptr())
    _lib.check(rc, "fused_decode_prep")
    return sel, row, scores


def fused_decode_sdpa(q, window, row, pooled, sel, sinks, inv_freq, params, *, scale,
                      pool_rows_in_params: bool = False, workspace=None):
    """Attend one decode token over the window and selected pooled rows (reference :733).

    With ``pool_rows_in_params`` ``pooled`` is a capacity buffer and ``params`` is int32 ``[position,
    write_idx, rows in use]``; ids that name a row not in use are skipped like negative ones.

    Args:
        q: float16 ``[n_heads, 512]`` post-norm, pre-rope query heads.
        window: float16 ``[window_rows, 512]`` local KV buffer (pre-update).
        row: float16 ``[512]`` prepared KV row (``fused_decode_prep``).
        pooled: float16 ``[n_rows, 512]`` compressed pool rows.
        sel: int32 ``[topk]`` selected pool row ids.
        sinks: float16 ``[n_heads]`` per-head attention sinks.
        inv_freq: float32 ``[32]`` rope inverse frequencies.
        params: int32 ``[position, write_idx]``; the prepared row replaces
            ``window[write_idx]``.
        scale: softmax scale (``head_dim ** -0.5``).

    Returns:
        float16 ``[n_heads, 512]`` attention output after the inverse rope.
    """
    if q.ndim != 2 or int(q.shape[1]) != _HEAD_DIM or q.dtype != torch.float16:
        raise ValueError("q must be float16 [n_heads, 512]")
    n_heads = int(q.shape[0])
    if n_heads <= 0:
        raise ValueError("q must carry at least one head")
    if window.ndim != 2 or int(window.shape[1]) != _HEAD_DIM or window.dtype != torch.float16:
        raise ValueError("window must be float16 [window_rows, 512]")
    if tuple(int(v) for v in row.shape) != (_HEAD_DIM,) or row.dtype != torch.float16:
        raise ValueError("row must be float16 [512]")
    if pooled.ndim != 2 or int(pooled.shape[1]) != _HEAD_DIM or pooled.dtype != torch.float16:
        raise ValueError("pooled must be float16 [n_rows, 512]")
    if sel.ndim != 1 or sel.dtype != torch.int32:
        raise ValueError("sel must be int32 [topk]")
    if tuple(int(v) for v in sinks.shape) != (n_heads,) or sinks.dtype != torch.float16:
        raise ValueError("sinks must be float16 [n_heads]")
    if int(inv_freq.shape[-1]) != _ROPE_DIM // 2 or inv_freq.dtype != torch.float32:
        raise ValueError("inv_freq must be float32 [32]")
    if params.dtype != torch.int32 or params.numel() < 2:
        raise ValueError("params must be int32 [position, write_idx]")
    if pool_rows_in_params and params.numel() < 3:
        raise ValueError("params must be int32 [position, write_idx, pool_rows] for a fixed-capacity pool")
    dev = _lib.require_device(q, window, row, pooled, sel, sinks, inv_freq, params)
    window_rows = int(window.shape[0])
    n_rows = int(pooled.shape[0])
    n_sel = int(sel.shape[0])
    qc, wc, rc_, pc = q.contiguous(), window.contiguous(), row.contiguous(), pooled.contiguous()
    sc, kc, fc, prm = sel.contiguous(), sinks.contiguous(), inv_freq.reshape(-1).contiguous(), params.reshape(-1).contiguous()
    out = torch.empty((n_heads, _HEAD_DIM), dtype=torch.float16, device=dev)
    ws = workspace if workspace is not None else _lib.sparse_attention_workspace(1, n_heads, window_rows + n_sel, dev)
    entry = _lib.lib().mspr_fused_decode_sdpa_fixed if pool_rows_in_params else _lib.lib().mspr_fused_decode_sdpa
    rc = entry(
        _lib.ptr(qc), n_heads, _lib.ptr(wc), window_rows, _lib.ptr(rc_), _lib.ptr(pc), n_rows, _lib.ptr(sc),
        n_sel, _lib.ptr(kc), _lib.ptr(fc), _lib.ptr(prm), float(scale), _lib.ptr(out), _lib.ptr(ws),
        ws.numel() * 4, _lib.stream_ptr())
    _lib.check(rc, "fused_decode_sdpa")
    return out


def fused_decode_enabled() -> bool:
    """Whether the fused decode island may engage (gate plus device; reference :789)."""
    return _ENABLED and _metal_available()
