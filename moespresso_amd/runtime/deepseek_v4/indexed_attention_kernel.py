"""DS4 indexed (gathered) mixed attention on MI355X.

Mirror of the reference module
``src/moespresso/runtime/deepseek_v4/indexed_attention_kernel.py`` for the
one-token decode consumer, plus the batched multi-head-latent form of the
BASELINE configuration (576-wide K, 512-wide V, bf16, batch > 1).

Visit rules of the decode consumer (reference kernel source, :120-173): ring
rows for positions ``[max(first_raw, pos0+1-window), pos0]`` at
``(raw_start + logical) % raw_cap``; then ``topk`` ids in order, where a
negative id is skipped and the first id ``>= min((pos0+1)//ratio, n_comp)``
ends the walk; K == V; scale ``512**-0.5``; the per-head sink joins the max and
the denominator once; an empty softmax gives zeros.

The reference walks the rows serially with one 32-lane group per head. Here a
workgroup owns a slice of the row list for all heads, K rows are read once into
LDS, the 64-head contraction runs on MFMA, and slices are merged by
log-sum-exp in a second launch.
"""

from __future__ import annotations

import torch

from moespresso_amd import _lib

_HEAD_DIM = 512


def indexed_mixed_attention_decode(q, raw_kv, comp_kv, topk, sinks, *, pos0: int, window: int = 128,
                                   ratio: int = 4, raw_start: int = 0):
    """One-token DS4 indexed mixed attention (reference :1496).

    Args:
        q: float32 ``[n_heads, 512]`` query heads (rounded to half on load).
        raw_kv: float16 ``[raw_cap, 512]`` contiguous/circular raw KV rows.
        comp_kv: float16 ``[n_comp, 512]`` compressed KV rows.
        topk: int32 ``[top_k]`` selected compressed row ids (other integer
            dtypes are cast, as in the reference).
        sinks: float32 ``[n_heads]`` attention sink logits (cast if needed).

    Returns:
        float32 ``[n_heads, 512]``.
    """
    if q.ndim != 2 or raw_kv.ndim != 2 or comp_kv.ndim != 2:
        raise ValueError("q, raw_kv, and comp_kv must be rank-2")
    n_heads = int(q.shape[0])
    head_dim = int(q.shape[1])
    if head_dim != _HEAD_DIM:
        raise ValueError("DS4 indexed attention probe currently requires head_dim=512")
    if int(raw_kv.shape[1]) != head_dim or int(comp_kv.shape[1]) != head_dim:
        raise ValueError("raw_kv and comp_kv width must match q")
    if topk.ndim != 1:
        raise ValueError("topk must be rank-1")
    if tuple(sinks.shape) != (n_heads,):
        raise ValueError("sinks must have shape [n_heads]")
    if q.dtype != torch.float32:
        raise ValueError("q must be float32, matching DS4-c's q buffer contract")
    if raw_kv.dtype != torch.float16 or comp_kv.dtype != torch.float16:
        raise ValueError("raw_kv and comp_kv must be float16")
    if topk.dtype != torch.int32:
        topk = topk.to(torch.int32)
    if sinks.dtype != torch.float32:
        sinks = sinks.to(torch.float32)
    raw_cap = int(raw_kv.shape[0])
    if raw_cap <= 0:
        raise ValueError("raw_kv must contain at least one row")
    if not (0 <= int(raw_start) < raw_cap):
        raise ValueError("raw_start must be inside raw_kv")
    n_comp = int(comp_kv.shape[0])
    if n_comp <= 0:
        raise ValueError("comp_kv must contain at least one row")
    dev = _lib.require_device(q, raw_kv, comp_kv, topk, sinks)
    top_k = int(topk.shape[0])
    qc, rc_, cc, tc, sc = (t.contiguous() for t in (q, raw_kv, comp_kv, topk, sinks))
    out = torch.empty((n_heads, head_dim), dtype=torch.float32, device=dev)
    ws = _lib.sparse_attention_workspace(1, n_heads, raw_cap + top_k, dev)
    rc = _lib.lib().mspr_indexed_mixed_attention_decode(
        _lib.ptr(qc), n_heads, _lib.ptr(rc_), raw_cap, _lib.ptr(cc), n_comp, _lib.ptr(tc), top_k,
        _lib.ptr(sc), int(pos0), int(window), int(ratio), int(raw_start), _lib.ptr(out), _lib.ptr(ws),
        ws.numel() * 4, _lib.stream_ptr())
    _lib.check(rc, "indexed_mixed_attention_decode")
    return out


def sparse_mla_decode(q, kv, rows, *, scale: float, v_dim: int = 512, window_start: int | None = None,
                      window_rows: int = 0, sinks=None, workspace=None, row_mul: int = 1, row_add: int = 0):
    """Batched sparse multi-head-latent decode attention (BASELINE config 5 shape).

    Every head of batch entry ``b`` attends ``kv[b, rows[b, i]]`` for each
    gathered id plus the contiguous window ``kv[b, window_start : window_start
    + window_rows]``. K is the whole row, V its first ``v_dim`` columns. The
    batched extension of ``indexed_mixed_attention_decode``; the reference
    callable serves batch 1, 512-wide float16 rows only.

    Args:
        q: ``[batch, n_heads, k_dim]`` float16 or bfloat16, ``k_dim`` 512 or 576.
        kv: ``[batch, n_pool, k_dim]`` same dtype.
        rows: int32 ``[batch, n_rows]`` gathered ids; the pool row of an id is
            ``id * row_mul + row_add`` (so compressed-entry ids of a ratio-4
            indexer address a per-token cache with ``row_mul=4, row_add=3``).
            Negative ids and rows outside the pool are skipped.
        scale: softmax scale.
        sinks: optional float32 ``[n_heads]`` sink logits.
        workspace: optional float32 scratch from a previous call of the same shape.

    Returns:
        ``[batch, n_heads, v_dim]`` in the input dtype.
    """
    if q.ndim != 3 or kv.ndim != 3 or rows.ndim != 2:
        raise ValueError("q must be [batch, n_heads, k_dim], kv [batch, n_pool, k_dim], rows [batch, n_rows]")
    batch, n_heads, k_dim = (int(v) for v in q.shape)
    if k_dim not in (512, 576):
        raise ValueError("k_dim must be 512 or 576")
    if int(v_dim) != 512:
        raise ValueError("v_dim must be 512")
    if q.dtype not in (torch.float16, torch.bfloat16) or kv.dtype != q.dtype:
        raise ValueError("q and kv must both be float16 or both be bfloat16")
    if int(kv.shape[0]) != batch or int(kv.shape[2]) != k_dim:
        raise ValueError("kv must have shape [batch, n_pool, k_dim]")
    if int(rows.shape[0]) != batch:
        raise ValueError("rows must have shape [batch, n_rows]")
    if rows.dtype != torch.int32:
        raise ValueError("rows must be int32")
    if not 1 <= n_heads <= 128:
        raise ValueError("n_heads must be between 1 and 128")
    n_pool = int(kv.shape[1])
    n_rows = int(rows.shape[1])
    window_rows = int(window_rows)
    win_start = 0 if window_start is None else int(window_start)
    if window_rows < 0 or (window_rows > 0 and not (0 <= win_start and win_start + window_rows <= n_pool)):
        raise ValueError("window must lie inside the pool")
    if sinks is not None:
        if tuple(sinks.shape) != (n_heads,):
            raise ValueError("sinks must have shape [n_heads]")
        if sinks.dtype != torch.float32:
            sinks = sinks.to(torch.float32)
        sinks = sinks.contiguous()
    dev = _lib.require_device(q, kv, rows, sinks)
    qc, kc, rc_ = q.contiguous(), kv.contiguous(), rows.contiguous()
    out = torch.empty((batch, n_heads, 512), dtype=q.dtype, device=dev)
    ws = workspace if workspace is not None else _lib.sparse_attention_workspace(batch, n_heads, n_rows + window_rows, dev)
    rc = _lib.lib().mspr_sparse_mla_decode(
        _lib.ptr(qc), _lib.ptr(kc), _lib.ptr(rc_), _lib.ptr(sinks), _lib.DTYPE_CODE[q.dtype], batch, n_heads,
        k_dim, 512, n_pool, n_rows, int(row_mul), int(row_add), win_start, window_rows, float(scale), _lib.ptr(out), _lib.ptr(ws),
        ws.numel() * 4, _lib.stream_ptr())
    _lib.check(rc, "sparse_mla_decode")
    return out
