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

import os

import torch

from moespresso_amd import _lib

_HEAD_DIM = 512

# Prefill consumer engagement counts by the variant the reference would have dispatched
# (reference :34-48). One HIP kernel serves all three; the names record the dispatch decision so
# A/B harnesses that read the counters keep working.
_CONSUMER_CALL_COUNTS = {"mma": 0, "v2": 0, "v1": 0}
_SCORES_TILED_CALL_COUNTS = {"f16": 0, "f32": 0}


def prefill_consumer_call_counts() -> dict[str, int]:
    """Return prefill consumer engagement counts by kernel variant (reference :41)."""
    return dict(_CONSUMER_CALL_COUNTS)


def indexer_scores_call_counts() -> dict[str, int]:
    """Return tiled score kernel engagement counts by operand dtype (reference :46)."""
    return dict(_SCORES_TILED_CALL_COUNTS)


def indexer_score_operands(q, index_comp):
    """Return the tiled score kernel operand pair in float32 (reference :51)."""
    return q.to(torch.float32), index_comp.to(torch.float32)


def _prefill_live_v2_enabled() -> bool:
    """Gate of the reference's 32-heads-per-threadgroup consumer, read per call (reference :1401)."""
    return os.environ.get("MOESPRESSO_DSV4_R4_PREFILL_CONSUMER_V2", "1") != "0"


def _prefill_live_mma_enabled() -> bool:
    """Gate of the reference's matrix-unit consumer, read per call (reference :1431)."""
    return os.environ.get("MOESPRESSO_DSV4_R4_PREFILL_CONSUMER_MMA", "1") != "0"


def _indexer_q_qat_v2_enabled() -> bool:
    """Gate of the reference's shuffle-based QAT restructure (bit-identical math, reference :1982)."""
    return os.environ.get("MOESPRESSO_DSV4_R4_PREFILL_QAT_V2", "1") != "0"


def indexed_mixed_attention_decode(q, raw_kv, comp_kv, topk, sinks, *, pos0: int, window: int = 128,
                                   ratio: int = 4, raw_start: int = 0):
    """Decode consumer of the indexed mixed attention: one query token (reference :1496).

    Operands: ``q`` is ``[n_heads, 512]`` float32 and is rounded to half precision when loaded;
    ``raw_kv`` ``[raw_cap, 512]`` float16 is the sliding-window ring, whose oldest row sits at
    ``raw_start``; ``comp_kv`` ``[n_comp, 512]`` float16 is the compressed pool; ``topk`` ``[top_k]``
    names the pool rows to visit (any integer type, converted to int32 as the reference does);
    ``sinks`` ``[n_heads]`` holds one sink logit per head (converted to float32 if needed).
    The result is float32 ``[n_heads, 512]``.
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


def _run_prefill(q, raw_kv, comp_kv, topk, sinks, *, batch, n_heads, n_tokens, strides, raw_cap, n_comp, pos0,
                 window, ratio, raw_start):
    """Launch the per-token indexed attention over tensors already validated; ``strides`` are the
    (batch, head, token) element strides of ``q`` and of the float32 output."""
    dev = _lib.require_device(q, raw_kv, comp_kv, topk, sinks)
    top_k = int(topk.shape[-1])
    out = torch.empty(q.shape, dtype=torch.float32, device=dev)
    max_win = min(int(window), raw_cap) if int(window) != 0 else raw_cap
    ws = _lib.prefill_attention_workspace(q.dtype, batch, n_heads, n_tokens, max_win, top_k, dev)
    rc = _lib.lib().mspr_indexed_mixed_attention_prefill(
        _lib.ptr(q), _lib.DTYPE_CODE[q.dtype], batch, n_heads, n_tokens, strides[0], strides[1], strides[2],
        _lib.ptr(raw_kv), raw_cap, _lib.ptr(comp_kv), n_comp, _lib.ptr(topk) if top_k else None, top_k,
        _lib.ptr(sinks), int(pos0), int(window), int(ratio), int(raw_start), _lib.ptr(out), _lib.ptr(ws),
        ws.numel() * 4, _lib.stream_ptr())
    _lib.check(rc, "indexed_mixed_attention_prefill")
    return out


def indexed_mixed_attention_prefill(q, raw_kv, comp_kv, topk, sinks, *, pos0: int, window: int = 128,
                                    ratio: int = 4, raw_start: int = 0):
    """Prefill consumer on token-major operands: the decode rules applied to every token of a chunk
    (reference :2030).

    Token ``t`` sits at position ``pos0 + t``. ``q`` is ``[tokens, n_heads, 512]`` float32; the ring
    ``raw_kv`` ``[raw_cap, 512]`` float16 ends with the row of the chunk's last token (position
    ``pos0 + tokens - 1``); ``comp_kv`` ``[n_comp, 512]`` float16 is the compressed pool; row ``t`` of
    ``topk`` ``[tokens, top_k]`` lists the pool rows of token ``t``; ``sinks`` ``[n_heads]`` are the
    per-head sink logits. The result is float32 with the shape of ``q``.
    """
    if q.ndim != 3 or raw_kv.ndim != 2 or comp_kv.ndim != 2:
        raise ValueError("q must be rank-3 and raw_kv/comp_kv rank-2")
    n_tokens, n_heads, head_dim = int(q.shape[0]), int(q.shape[1]), int(q.shape[2])
    if n_tokens <= 0:
        raise ValueError("q must contain at least one token")
    if head_dim != _HEAD_DIM:
        raise ValueError("DS4 indexed prefill probe currently requires head_dim=512")
    if n_heads % 8 != 0:
        raise ValueError("DS4 indexed prefill probe requires n_heads to be divisible by 8")
    if int(raw_kv.shape[1]) != head_dim or int(comp_kv.shape[1]) != head_dim:
        raise ValueError("raw_kv and comp_kv width must match q")
    if topk.ndim != 2 or int(topk.shape[0]) != n_tokens:
        raise ValueError("topk must have shape [tokens, top_k]")
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
    if int(comp_kv.shape[0]) <= 0:
        raise ValueError("comp_kv must contain at least one row")
    return _run_prefill(q.contiguous(), raw_kv.contiguous(), comp_kv.contiguous(), topk.contiguous(),
                        sinks.contiguous(), batch=1, n_heads=n_heads, n_tokens=n_tokens,
                        strides=(0, head_dim, n_heads * head_dim), raw_cap=raw_cap, n_comp=int(comp_kv.shape[0]),
                        pos0=pos0, window=window, ratio=ratio, raw_start=raw_start)


def _validate_live(q, raw_kv, comp_kv, topk, sinks, q_dtype, q_dtype_message, raw_start):
    if q.ndim != 4 or raw_kv.ndim != 4 or comp_kv.ndim != 3:
        raise ValueError("q/raw_kv/comp_kv must have live BHLD/B1LD/BPD layouts")
    batch, n_heads, n_tokens, head_dim = (int(v) for v in q.shape)
    if batch <= 0 or n_tokens <= 0:
        raise ValueError("q must contain at least one batch and token")
    if head_dim != _HEAD_DIM:
        raise ValueError("DS4 indexed prefill probe currently requires head_dim=512")
    if n_heads % 8 != 0:
        raise ValueError("DS4 indexed prefill probe requires n_heads to be divisible by 8")
    if int(raw_kv.shape[0]) != batch or int(comp_kv.shape[0]) != batch:
        raise ValueError("raw_kv and comp_kv batch size must match q")
    if int(raw_kv.shape[-1]) != head_dim or int(comp_kv.shape[-1]) != head_dim:
        raise ValueError("raw_kv and comp_kv width must match q")
    if topk.ndim != 3 or int(topk.shape[0]) != batch or int(topk.shape[1]) != n_tokens:
        raise ValueError("topk must have shape [batch, tokens, top_k]")
    if tuple(sinks.shape) != (n_heads,):
        raise ValueError("sinks must have shape [n_heads]")
    if q.dtype != q_dtype:
        raise ValueError(q_dtype_message)
    if raw_kv.dtype != torch.float16 or comp_kv.dtype != torch.float16:
        raise ValueError("raw_kv and comp_kv must be float16")
    raw_cap = int(raw_kv.shape[2])
    if raw_cap <= 0:
        raise ValueError("raw_kv must contain at least one row")
    if not (0 <= int(raw_start) < raw_cap):
        raise ValueError("raw_start must be inside raw_kv")
    if int(raw_kv.shape[1]) != 1:
        raise ValueError("q/raw_kv/comp_kv must have live BHLD/B1LD/BPD layouts")
    if int(comp_kv.shape[1]) <= 0:
        raise ValueError("comp_kv must contain at least one row")
    return batch, n_heads, n_tokens, head_dim, raw_cap


def _count_live_dispatch(n_heads: int) -> None:
    # the reference's selection order (:1645-1676): mma for heads % 16 == 0, then v2 for % 32, else v1
    if n_heads % 16 == 0 and _prefill_live_mma_enabled():
        _CONSUMER_CALL_COUNTS["mma"] += 1
    elif n_heads % 32 == 0 and _prefill_live_v2_enabled():
        _CONSUMER_CALL_COUNTS["v2"] += 1
    else:
        _CONSUMER_CALL_COUNTS["v1"] += 1


def _launch_live(q, raw_kv, comp_kv, topk, sinks, dims, *, pos0, window, ratio, raw_start):
    batch, n_heads, n_tokens, head_dim, raw_cap = dims
    if topk.dtype != torch.int32:
        topk = topk.to(torch.int32)
    if sinks.dtype != torch.float32:
        sinks = sinks.to(torch.float32)
    return _run_prefill(q.contiguous(), raw_kv.contiguous(), comp_kv.contiguous(), topk.contiguous(),
                        sinks.contiguous(), batch=batch, n_heads=n_heads, n_tokens=n_tokens,
                        strides=(n_heads * n_tokens * head_dim, n_tokens * head_dim, head_dim), raw_cap=raw_cap,
                        n_comp=int(comp_kv.shape[1]), pos0=pos0, window=window, ratio=ratio, raw_start=raw_start)


def indexed_mixed_attention_prefill_live_f16(q, raw_kv, comp_kv, topk, sinks, *, pos0: int, window: int = 128,
                                             ratio: int = 4, raw_start: int = 0):
    """The prefill consumer on the layouts the attention block holds, half-precision queries (reference :1571).

    ``q`` is head-major ``[batch, n_heads, tokens, 512]`` float16, the ring ``[batch, 1, raw_cap, 512]``
    and the pool ``[batch, n_comp, 512]`` float16, ``topk`` ``[batch, tokens, top_k]`` int32 and ``sinks``
    ``[n_heads]`` float32; the float32 result has the shape of ``q``.
    """
    dims = _validate_live(q, raw_kv, comp_kv, topk, sinks, torch.float16,
                          "live prefill probe requires q to be float16", raw_start)
    _count_live_dispatch(dims[1])
    return _launch_live(q, raw_kv, comp_kv, topk, sinks, dims, pos0=pos0, window=window, ratio=ratio,
                        raw_start=raw_start)


def indexed_mixed_attention_prefill_live_f32(q, raw_kv, comp_kv, topk, sinks, *, pos0: int, window: int = 128,
                                             ratio: int = 4, raw_start: int = 0):
    """Indexed prefill attention on the live BHLD layout, float32 queries rounded to half on load
    (reference :1679)."""
    dims = _validate_live(q, raw_kv, comp_kv, topk, sinks, torch.float32,
                          "live f32 prefill probe requires q to be float32", raw_start)
    _count_live_dispatch(dims[1])
    return _launch_live(q, raw_kv, comp_kv, topk, sinks, dims, pos0=pos0, window=window, ratio=ratio,
                        raw_start=raw_start)


def banded_prefill_attention_live(q, raw_kv, comp_kv, topk, sinks, *, pos0: int, window: int, ratio: int):
    """Banded prefill attention: a ``window``-token local band plus every visible pooled row (reference :1782).

    ``topk`` carries ascending pool row ids, so the visibility rule (id below ``(position+1)/ratio``)
    reproduces the compressed-pool predicate. Zero-pool layers pass a one-row ``comp_kv`` with a
    zero-width ``topk``.
    """
    if q.ndim != 4 or raw_kv.ndim != 4 or comp_kv.ndim != 3:
        raise ValueError("q/raw_kv/comp_kv must have live BHLD/B1LD/BPD layouts")
    batch, n_heads, n_tokens, head_dim = (int(v) for v in q.shape)
    if batch <= 0 or n_tokens <= 0:
        raise ValueError("q must contain at least one batch and token")
    if head_dim != _HEAD_DIM:
        raise ValueError("banded mma attention requires head_dim=512")
    if n_heads % 16 != 0 or not _prefill_live_mma_enabled():
        raise ValueError("banded mma attention requires the mma consumer")
    if int(raw_kv.shape[0]) != batch or int(comp_kv.shape[0]) != batch:
        raise ValueError("raw_kv and comp_kv batch size must match q")
    if int(raw_kv.shape[-1]) != head_dim or int(comp_kv.shape[-1]) != head_dim:
        raise ValueError("raw_kv and comp_kv width must match q")
    if int(comp_kv.shape[1]) <= 0:
        raise ValueError("comp_kv must contain at least one row")
    if topk.ndim != 3 or int(topk.shape[0]) != batch or int(topk.shape[1]) != n_tokens:
        raise ValueError("topk must have shape [batch, tokens, width]")
    if q.dtype not in (torch.float16, torch.float32):
        raise ValueError("banded mma attention requires q to be float16 or float32")
    if raw_kv.dtype != torch.float16 or comp_kv.dtype != torch.float16:
        raise ValueError("raw_kv and comp_kv must be float16")
    if int(window) <= 0 or int(ratio) <= 0:
        raise ValueError("banded mma attention requires positive window and ratio")
    if tuple(sinks.shape) != (n_heads,):
        raise ValueError("sinks must have shape [n_heads]")
    raw_cap = int(raw_kv.shape[2])
    if raw_cap <= 0:
        raise ValueError("raw_kv must contain at least one row")
    dims = (batch, n_heads, n_tokens, head_dim, raw_cap)
    return _launch_live(q, raw_kv, comp_kv, topk, sinks, dims, pos0=pos0, window=window, ratio=ratio, raw_start=0)


def indexer_scores_tiled_live(q, weights, index_comp, *, pos0: int, ratio: int = 4):
    """Ratio-4 indexer scores over a prefill chunk (reference :1888).

    Args:
        q: float32 or float16 ``[batch, n_heads, tokens, 128]`` QAT indexer queries (staged as half).
        weights: float32 ``[batch, tokens, n_heads]`` head weights including the DS4 scale factors.
        index_comp: ``[batch, n_comp, 128]`` QAT compressed index rows, same dtype as ``q``.

    Returns:
        float32 ``[batch, tokens, n_comp]``, ``-inf`` where the row is not yet visible to the token.
    """
    if q.ndim != 4 or weights.ndim != 3 or index_comp.ndim != 3:
        raise ValueError("q, weights, and index_comp must be BHLD/BLH/BPD")
    batch, n_heads, n_tokens, head_dim = (int(v) for v in q.shape)
    n_comp = int(index_comp.shape[1])
    if batch <= 0 or n_tokens <= 0:
        raise ValueError("q must contain at least one batch and token")
    if head_dim != 128:
        raise ValueError("DS4 indexer score probe requires head_dim=128")
    if int(index_comp.shape[0]) != batch or int(index_comp.shape[2]) != head_dim:
        raise ValueError("index_comp must have shape [batch, n_comp, 128]")
    if tuple(weights.shape) != (batch, n_tokens, n_heads):
        raise ValueError("weights must have shape [batch, tokens, n_heads]")
    if weights.dtype != torch.float32:
        raise ValueError("weights must be float32")
    if q.dtype == torch.float16 or index_comp.dtype == torch.float16:
        if q.dtype != torch.float16 or index_comp.dtype != torch.float16:
            raise ValueError("half score operands require both q and index_comp as float16")
        operand_form = "f16"
    elif q.dtype == torch.float32 and index_comp.dtype == torch.float32:
        operand_form = "f32"
    else:
        raise ValueError("q and index_comp must both be float32 or both be float16")
    if n_comp <= 0:
        raise ValueError("index_comp must contain at least one compressed row")
    if n_heads > 64:
        raise ValueError("DS4 indexer score probe supports between 1 and 64 heads")
    dev = _lib.require_device(q, weights, index_comp)
    _SCORES_TILED_CALL_COUNTS[operand_form] += 1
    qc, wc, cc = q.contiguous(), weights.contiguous(), index_comp.contiguous()
    scores = torch.empty((batch, n_tokens, n_comp), dtype=torch.float32, device=dev)
    rc = _lib.lib().mspr_indexer_scores_tiled_live(
        _lib.ptr(qc), _lib.ptr(wc), _lib.ptr(cc), _lib.DTYPE_CODE[qc.dtype], batch, n_heads, n_tokens, n_comp,
        int(pos0), int(ratio), _lib.ptr(scores), _lib.stream_ptr())
    _lib.check(rc, "indexer_scores_tiled_live")
    return scores


def indexer_q_qat_live(q):
    """Hadamard-128 + FP4 QAT of live BHLD query rows, prefill-side rules (reference :1989)."""
    if q.ndim != 4:
        raise ValueError("q must have shape [batch, n_heads, tokens, 128]")
    batch, n_heads, n_tokens, head_dim = (int(v) for v in q.shape)
    if batch <= 0 or n_tokens <= 0:
        raise ValueError("q must contain at least one batch and token")
    if head_dim != 128:
        raise ValueError("DS4 indexer QAT probe requires head_dim=128")
    if q.dtype != torch.float32:
        raise ValueError("q must be float32")
    dev = _lib.require_device(q)
    qc = q.contiguous()
    out = torch.empty(qc.shape, dtype=torch.float32, device=dev)
    rc = _lib.lib().mspr_indexer_q_qat_live(_lib.ptr(qc), batch * n_heads * n_tokens, _lib.ptr(out),
                                            _lib.stream_ptr())
    _lib.check(rc, "indexer_q_qat_live")
    return out


def _composed_sink_attention(qh, rows, sinks_h):
    """softmax(q . rows^T / sqrt(D), with one sink logit per head in the denominator) . rows, float32:
    the composition that ``scaled_dot_product_attention(..., sinks=)`` computes in the reference forms."""
    head_dim = int(qh.shape[-1])
    if int(rows.shape[0]) == 0:
        return torch.zeros(qh.shape, dtype=torch.float32, device=qh.device)
    logits = (qh.float() @ rows.float().T) * (float(head_dim) ** -0.5)
    full = torch.cat([logits, sinks_h.float()[:, None]], dim=1)
    prob = torch.softmax(full, dim=1)[:, :-1]
    return prob @ rows.float()


def mlx_selected_rows_attention_reference(q, raw_kv, comp_kv, topk, sinks):
    """Composed selected-row consumer kept as correctness and speed reference (reference :2111).

    Every ring row, then ``comp_kv[topk]``, attended by float16 ``q`` with float16 sinks; no visibility
    rules. Built from tensor operations on the device (the reference composes MLX operations the same
    way): it is the form the kernels are compared with, not a kernel path. The name is the reference's.
    """
    selected = torch.index_select(comp_kv, 0, topk.to(torch.int64))
    full = torch.cat([raw_kv, selected], dim=0)
    return _composed_sink_attention(q.to(torch.float16), full, sinks.to(torch.float16)).reshape(q.shape)


def mlx_indexed_mixed_attention_prefill_reference(q, raw_kv, comp_kv, topk, sinks, *, pos0: int, window: int = 128,
                                                  ratio: int = 4):
    """Composed per-token reference of the prefill consumer (reference :2133).

    Token ``t`` attends the ring rows of positions ``[max(first_raw, pos0+t+1-window), pos0+t]`` (ring
    starting at row 0) and the pool rows whose ids lie in ``[0, (pos0+t+1)//ratio)`` — ids outside that
    range are dropped wherever they stand, where the kernel stops at the first one. q ``[tokens,
    n_heads, 512]``; result float32 of the same shape.
    """
    n_tokens, n_heads, head_dim = (int(v) for v in q.shape)
    n_raw = int(raw_kv.shape[0])
    raw_last_pos = int(pos0) + n_tokens - 1
    first_raw_pos = raw_last_pos + 1 - n_raw
    sinks_h = sinks.to(torch.float16)
    rows_out = []
    for token in range(n_tokens):
        qpos = int(pos0) + token
        window_first = qpos + 1 - int(window) if window and qpos + 1 > window else 0
        first = max(first_raw_pos, window_first)
        last = min(qpos, raw_last_pos)
        parts = []
        if first <= last:
            parts.append(raw_kv[first - first_raw_pos:last - first_raw_pos + 1])
        visible = min((qpos + 1) // int(ratio), int(comp_kv.shape[0]))
        ids = topk[token].to(torch.int64)
        ids = ids[(ids >= 0) & (ids < visible)]
        if int(ids.numel()):
            parts.append(torch.index_select(comp_kv, 0, ids))
        full = torch.cat(parts, dim=0) if parts else raw_kv[:0]
        rows_out.append(_composed_sink_attention(q[token].to(torch.float16), full, sinks_h))
    return torch.stack(rows_out, dim=0)
