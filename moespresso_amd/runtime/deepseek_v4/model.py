"""DS4 attention-layer glue around the decode kernels: cache write path, pooled-row QAT
maintenance, the decode score contract and the fused ratio-4 decode attention wrapper.

Mirror of the attention-path pieces of the reference module
``src/moespresso/runtime/deepseek_v4/model.py``:

- ``_dsv4_indexer_qat`` (:745) and ``_dsv4_decode_indexer_qat`` (:772): indexer QAT of 128-wide rows;
- ``_deepseek_v4_fp8_kv_roundtrip`` (:559): E4M3FN round trip of the non-rope prefix of KV rows;
- ``_cache_with_fp8_kv_roundtrip`` (:395) / ``_update_and_fetch_with_fp8_kv`` (:381): the cache write
  path that rounds rows on append; ``_cache_with_compressed_pool_aux_trim_clear`` (:416);
- ``pooled_qat_update``: the incremental pooled-row QAT cache shared by the score contract (:925-944)
  and the fused decode wrapper (:1707-1723);
- ``_IndexerDS4ScoreContract`` (:833): the decode-shaped branch (QAT'd query and pool, fused score
  row, deterministic top-k);
- ``_Ratio4DecodeFusedAttention`` (:1519): eligibility (:1551-1607), the two fused launches and the
  direct ring append (:1756-1789);
- ``_Ratio4PrefillFastAttention`` (:1305): the prefill chunk through the live-layout kernels.

The wrapped blocks are the model's own modules (torch here). Everything outside the fused contract
goes to the wrapped block: an ineligible call is the block's own ``__call__``; a call that fails a
late check finishes through the block's ``composed_decode_tail`` when it has one. This package ships
no composed attention of its own.
"""

from __future__ import annotations

import os
from types import MethodType

import torch

from moespresso_amd.runtime.deepseek_v4 import attention_seam_kernel as _seam
from moespresso_amd.runtime.deepseek_v4 import decode_attention_kernel, indexer_score_kernel

_CACHE_WRAPPER_ORIGINALS_ATTR = "_moespresso_dsv4_cache_wrapper_originals"
_DSV4_DECODE_QAT_KERNEL_ENV = "MOESPRESSO_DSV4_INDEXER_DECODE_QAT_KERNEL"


class DeepseekV4RuntimeLoadError(RuntimeError):
    """Shape contract of the DS4 runtime violated (name kept from the reference)."""


# ---------------------------------------------------------------- row transforms

def _rows_argument(args, name: str) -> torch.Tensor:
    """The reference's row helpers take its array-library module as a leading positional (``f(mx, x)``);
    both ``f(x)`` and ``f(module, x)`` are accepted here and the module handle is ignored."""
    if len(args) == 1:
        return args[0]
    if len(args) == 2 and not isinstance(args[0], torch.Tensor):
        return args[1]
    raise TypeError(f"{name} takes the rows, optionally behind an array-module handle")


def _dsv4_indexer_qat(*args) -> torch.Tensor:
    """Hadamard-128 + e2m1 activation round trip of 128-wide rows, float32 out (reference :745)."""
    return indexer_score_kernel.indexer_qat_rows(_rows_argument(args, "_dsv4_indexer_qat"))


def _dsv4_decode_indexer_qat(*args):
    """Decode-side QAT; returns ``(rows, used_kernel)`` (reference :772).

    There is one implementation here, the kernel; the kill switch of the reference selects its composed
    chain, which computes the same bits, so it only changes the engagement flag.
    """
    used = os.environ.get(_DSV4_DECODE_QAT_KERNEL_ENV, "1") != "0"
    return indexer_score_kernel.indexer_qat_rows(_rows_argument(args, "_dsv4_decode_indexer_qat")), used


def _deepseek_v4_fp8_kv_roundtrip(x: torch.Tensor, *, head_dim: int = 512, rot_dim: int = 64) -> torch.Tensor:
    """E4M3FN round trip of the non-rope prefix of compressed-KV rows (reference :559).

    Rows whose last axis is not ``head_dim`` wide, and empty tensors, pass through. The arithmetic is
    float32 whatever the element type; the result is cast back.
    """
    if x.ndim == 0 or int(x.shape[-1]) != int(head_dim) or x.numel() == 0:
        return x
    n_nope = int(head_dim) - int(rot_dim)
    if n_nope <= 0:
        return x
    if n_nope % 64:
        raise DeepseekV4RuntimeLoadError("DeepSeek V4 compressed KV non-RoPE width must be divisible by 64")
    if int(head_dim) != 512 or int(rot_dim) != 64:
        raise DeepseekV4RuntimeLoadError("the E4M3FN row kernel serves head_dim 512 with a 64-wide rope tail")
    if x.dtype == torch.float32:
        return decode_attention_kernel.fp8_kv_prefix_rows(x)
    return decode_attention_kernel.fp8_kv_prefix_rows(x.to(torch.float32)).to(x.dtype)


# ---------------------------------------------------------------- cache write path

def _cache_wrapper_originals(cache) -> dict:
    """Per-cache record of the methods the wrappers below replaced (reference :363-378)."""
    originals = getattr(cache, _CACHE_WRAPPER_ORIGINALS_ATTR, None)
    if not isinstance(originals, dict):
        originals = {}
        object.__setattr__(cache, _CACHE_WRAPPER_ORIGINALS_ATTR, originals)
    return originals


def _update_and_fetch_with_fp8_kv(self, keys, values):
    original_update = getattr(self, _CACHE_WRAPPER_ORIGINALS_ATTR)["update_and_fetch"]
    rounded_keys = _deepseek_v4_fp8_kv_roundtrip(keys)
    rounded_values = rounded_keys if values is keys else _deepseek_v4_fp8_kv_roundtrip(values)
    return original_update(rounded_keys, rounded_values)


def _cache_with_fp8_kv_roundtrip(cache):
    """Round every appended KV row through E4M3FN; idempotent (reference :395-409)."""
    if getattr(cache, "_moespresso_dsv4_fp8_kv_cache", False):
        return cache
    _cache_wrapper_originals(cache)["update_and_fetch"] = cache.update_and_fetch
    object.__setattr__(cache, "update_and_fetch", MethodType(_update_and_fetch_with_fp8_kv, cache))
    object.__setattr__(cache, "_moespresso_dsv4_fp8_kv_cache", True)
    return cache


def _trim_with_compressed_pool_aux_clear(self, n):
    result = getattr(self, _CACHE_WRAPPER_ORIGINALS_ATTR)["trim"](n)
    for attr, keys in (("indexer_state", ("pooled_qat", "pooled_qat_rows")),
                       ("compressor_state", ("pooled_fp8", "pooled_fp8_rows"))):
        state = getattr(self, attr, None)
        if isinstance(state, dict):
            for key in keys:
                state.pop(key, None)
    return result


def _cache_with_compressed_pool_aux_trim_clear(cache):
    """Drop the derived pool caches whenever the cache is trimmed (reference :416-437)."""
    if getattr(cache, "_moespresso_dsv4_compressed_pool_aux_trim_clear", False):
        return cache
    original_trim = getattr(cache, "trim", None)
    if original_trim is None:
        return cache
    _cache_wrapper_originals(cache)["trim"] = original_trim
    object.__setattr__(cache, "trim", MethodType(_trim_with_compressed_pool_aux_clear, cache))
    object.__setattr__(cache, "_moespresso_dsv4_compressed_pool_aux_trim_clear", True)
    return cache


def pooled_qat_update(state, pooled: torch.Tensor):
    """QAT'd indexer pool rows, reusing what ``state`` already holds.

    Pool rows only ever append, so rows QAT'd on an earlier token are kept and only the new tail goes
    through the kernel (reference :925-944, :1707-1723). Returns ``(pooled_qat, cached_rows, new_rows)``
    and leaves the refreshed cache in ``state`` when it is a dict.
    """
    rows = int(pooled.shape[1])
    cached = state.get("pooled_qat") if isinstance(state, dict) else None
    cached_rows = int(state.get("pooled_qat_rows", 0) or 0) if isinstance(state, dict) else 0
    if cached is not None and 0 < cached_rows <= rows:
        if cached_rows == rows:
            return cached, cached_rows, 0
        tail = _dsv4_indexer_qat(pooled[:, cached_rows:, :])
        pooled_qat = torch.cat([cached, tail], dim=1)
        state["pooled_qat"] = pooled_qat
        state["pooled_qat_rows"] = rows
        return pooled_qat, cached_rows, rows - cached_rows
    pooled_qat = _dsv4_indexer_qat(pooled)
    if isinstance(state, dict):
        state["pooled_qat"] = pooled_qat
        state["pooled_qat_rows"] = rows
    return pooled_qat, 0, rows


# ---------------------------------------------------------------- decode score contract

class _IndexerDS4ScoreContract:
    """DS4 indexer QAT and top-k selection for one decode token (reference :833).

    The decode-shaped call (batch 1, one token) runs here: advance the indexer compressor, keep the
    QAT'd pool rows, project and rope the indexer queries, score every pool row in one launch and take
    the top-k. Every other shape goes to the wrapped indexer.
    """

    _COUNTERS = ("calls", "tokens", "pooled_rows", "topk_rows", "score_elements", "qat_elements",
                 "cached_pooled_rows", "new_qat_pooled_rows", "fused_score_calls", "decode_qat_kernel_calls")

    def __init__(self, original, compress_ratio: int, *, layer_index: int):
        self._original = original
        self._compress_ratio = int(compress_ratio)
        self._layer_index = int(layer_index)
        self._moespresso_dsv4_indexer_score_contract = True
        for name in self._COUNTERS:
            setattr(self, f"_moespresso_dsv4_indexer_score_contract_{name}", 0)

    def __getattr__(self, name: str):
        return getattr(self._original, name)

    def _bump(self, name: str, amount: int) -> None:
        key = f"_moespresso_dsv4_indexer_score_contract_{name}"
        setattr(self, key, getattr(self, key) + int(amount))

    def _engages(self, x) -> bool:
        """Everything that decides whether this call is served here, checked before any cache state moves:
        the decode shape, the score-kernel gate and the indexer geometry the kernel serves."""
        B, L, _ = x.shape
        if int(B) != 1 or int(L) != 1:
            return False
        if not indexer_score_kernel._ENABLED or not indexer_score_kernel._metal_available():
            return False
        ind = self._original
        if int(ind.head_dim) != 128 or not 1 <= int(ind.n_heads) <= 64:
            return False
        return x.dtype in (torch.float32, torch.float16, torch.bfloat16)

    def __call__(self, x, q_residual, rope, position_rope, cache, start_pos):
        # The wrapped indexer advances the stateful compressor itself, so it may only be entered while
        # this call has not: the decision is taken up front, and once the compressor has run the call is
        # finished here whatever the operands look like (the reference finishes inline as well, :1040-1056).
        if not self._engages(x):
            return self._original(x, q_residual, rope, position_rope, cache, start_pos)
        ind = self._original
        pooled = ind.compressor(x, rope, cache, start_pos, state_key="indexer_state")
        if int(pooled.shape[1]) == 0:
            return None
        pooled_rows = int(pooled.shape[1])
        heads, head_dim = int(ind.n_heads), int(ind.head_dim)
        topk_rows = min(int(ind.index_topk), pooled_rows)
        self._bump("calls", 1)
        self._bump("tokens", 1)
        self._bump("pooled_rows", pooled_rows)
        self._bump("topk_rows", topk_rows)
        self._bump("score_elements", heads * pooled_rows)
        q = ind.wq_b(q_residual).reshape(1, 1, heads, head_dim).transpose(1, 2)
        q = _seam.fused_partial_rope(q, position_rope.inv_freq, offset=int(start_pos))
        state = getattr(cache, "indexer_state", None)
        pooled_qat, cached_rows, new_rows = pooled_qat_update(state, pooled)
        self._bump("qat_elements", heads * head_dim + new_rows * head_dim)
        self._bump("cached_pooled_rows", cached_rows)
        self._bump("new_qat_pooled_rows", new_rows)
        weights = ind.weights_proj(x).to(torch.float32) * (heads ** -0.5)
        if q.dtype not in (torch.float32, torch.float16, torch.bfloat16):
            q = q.to(torch.float32)
        scores = indexer_score_kernel.fused_qat_indexer_scores(
            q, pooled_qat.to(torch.float32), weights.reshape(1, 1, heads), float(ind.scale))
        self._bump("fused_score_calls", 1)
        return indexer_score_kernel.topk_select(scores.reshape(1, 1, pooled_rows), topk_rows)


# ---------------------------------------------------------------- fused ratio-4 decode attention

class _Ratio4DecodeFusedAttention:
    """DS4 ratio-4 decode attention as two fused launches (reference :1519).

    Projections, norms and compressor calls stay with the wrapped block's own modules; the indexer
    query QAT, scoring, top-k and KV-row preparation run in ``fused_decode_prep``, rope + selected-row
    attention + inverse rope in ``fused_decode_sdpa``. The prepared KV row equals the composed
    rope + E4M3FN round trip bit for bit, so it is appended to the ring directly with the ring's own
    steady-state bookkeeping.
    """

    def __init__(self, original, *, cache_cls):
        self._original = original
        self._cache_cls = cache_cls
        self._moespresso_dsv4_fused_decode_attention = True
        self.fused_decode_calls = 0
        self.fused_decode_composed_tail_calls = 0
        self._fused_sinks_f16 = None

    def __getattr__(self, name: str):
        return getattr(self._original, name)

    def _decode_eligible(self, x, cache) -> bool:
        """The proven decode contract, checked before any cache mutation (reference :1551-1607)."""
        if not decode_attention_kernel.fused_decode_enabled():
            return False
        if os.environ.get("MOESPRESSO_DSV4_INDEXER_DUMP_PREFIX"):
            return False
        attn = self._original
        if x.ndim != 3 or int(x.shape[0]) != 1 or int(x.shape[1]) != 1:
            return False
        if x.dtype != torch.float16:
            return False
        if int(getattr(attn, "compress_ratio", 0) or 0) != 4:
            return False
        if not hasattr(attn, "indexer"):
            return False
        if int(attn.head_dim) != 512 or int(getattr(attn.rope, "dims", 0)) != 64:
            return False
        indexer = attn.indexer
        if int(indexer.head_dim) != 128 or not 0 < int(indexer.n_heads) <= 64:
            return False
        if int(indexer.index_topk) <= 0:
            return False
        if not isinstance(cache, self._cache_cls):
            return False
        # the prepared row bakes in the E4M3FN round trip: the cache must carry that contract for the
        # direct append to equal update_and_fetch
        if not getattr(cache, "_moespresso_dsv4_fp8_kv_cache", False):
            return False
        local = getattr(cache, "local", None)
        window = getattr(attn.args, "sliding_window", None)
        max_size = getattr(local, "max_size", None)
        if window is None or max_size is None or int(max_size) != int(window):
            return False
        if int(getattr(local, "keep", -1)) != 0:
            return False
        keys = getattr(local, "keys", None)
        values = getattr(local, "values", None)
        if keys is None or values is None:
            return False
        if int(local.offset) < int(max_size):
            return False
        expected = (1, 1, int(max_size), int(attn.head_dim))
        if tuple(int(v) for v in keys.shape) != expected or tuple(int(v) for v in values.shape) != expected:
            return False
        if keys.dtype != torch.float16 or values.dtype != torch.float16:
            return False
        return True

    def _composed_decode_tail(self, **kwargs):
        """Finish the token with the wrapped block's composed sequence (reference :1609-1651)."""
        tail = getattr(self._original, "composed_decode_tail", None)
        if tail is None:
            raise RuntimeError("the fused decode contract failed after the compressor advanced and the wrapped "
                               "block provides no composed_decode_tail to finish the token")
        self.fused_decode_composed_tail_calls += 1
        return tail(**kwargs)

    def __call__(self, x, mask=None, cache=None):
        if cache is None or not self._decode_eligible(x, cache):
            return self._original(x, mask=mask, cache=cache)

        attn = self._original
        indexer = attn.indexer
        local = cache.local
        offset = int(cache.offset)
        write_idx = int(local._idx)
        if write_idx == int(local.max_size):
            write_idx = int(local.keep)

        q_residual = attn.q_norm(attn.wq_a(x))
        q = attn.wq_b(q_residual).reshape(1, 1, attn.n_heads, attn.head_dim)
        q = torch.nn.functional.rms_norm(q, (int(attn.head_dim),), weight=None, eps=float(attn.args.rms_norm_eps))
        kv = attn.kv_norm(attn.wkv(x)).reshape(1, 1, 1, attn.head_dim)

        pooled = attn.compressor(x, attn.compress_rope, cache, offset)
        n_rows = int(pooled.shape[1])
        topk_width = int(indexer.index_topk)
        if (n_rows <= topk_width or n_rows >= (1 << 16) or pooled.dtype != torch.float16
                or q.dtype != torch.float16 or kv.dtype != torch.float16):
            return self._composed_decode_tail(x=x, q_residual=q_residual, q=q, kv=kv, pooled=pooled, cache=cache,
                                              offset=offset, run_indexer=True, topk=None)

        # indexer-side prep: advance the indexer compressor, keep the pooled QAT cache, project the
        # indexer queries and head weights
        index_pooled = indexer.compressor(x, attn.compress_rope, cache, offset, state_key="indexer_state")
        state = getattr(cache, "indexer_state", None)
        index_pooled_qat, _, _ = pooled_qat_update(state, index_pooled)
        index_rows = int(index_pooled.shape[1])

        q_idx = indexer.wq_b(q_residual).reshape(1, 1, indexer.n_heads, indexer.head_dim).transpose(1, 2)
        q_idx = _seam.fused_partial_rope(q_idx, attn.rope.inv_freq, offset=offset)
        weights = indexer.weights_proj(x).to(torch.float32) * (int(indexer.n_heads) ** -0.5)

        if index_rows != n_rows or q_idx.dtype not in (torch.float32, torch.float16, torch.bfloat16):
            # the indexer state already advanced: select with the standalone score kernel instead of
            # re-entering the wrapped indexer
            scores = indexer_score_kernel.fused_qat_indexer_scores(q_idx, index_pooled_qat, weights,
                                                                   float(indexer.scale))
            k = min(topk_width, index_rows)
            topk = indexer_score_kernel.topk_select(scores.reshape(1, 1, index_rows), k)
            return self._composed_decode_tail(x=x, q_residual=q_residual, q=q, kv=kv, pooled=pooled, cache=cache,
                                              offset=offset, run_indexer=False, topk=topk)

        params = torch.tensor([offset, write_idx], dtype=torch.int32, device=x.device)
        inv_freq = attn.rope.inv_freq
        sinks = self._fused_sinks_f16
        if sinks is None:
            sinks = attn.attn_sink.to(torch.float16)
            self._fused_sinks_f16 = sinks

        sel, row, _scores = decode_attention_kernel.fused_decode_prep(
            q_idx.reshape(int(indexer.n_heads), int(indexer.head_dim)),
            index_pooled_qat.reshape(n_rows, int(indexer.head_dim)),
            weights.reshape(int(indexer.n_heads)),
            kv.reshape(int(attn.head_dim)),
            inv_freq, params, scale=float(indexer.scale), topk=topk_width)
        heads = decode_attention_kernel.fused_decode_sdpa(
            q.reshape(int(attn.n_heads), int(attn.head_dim)),
            local.keys.reshape(int(local.max_size), int(attn.head_dim)),
            row,
            pooled.reshape(n_rows, int(attn.head_dim)),
            sel, sinks, inv_freq, params, scale=float(attn.softmax_scale))

        # append the prepared row with the ring's steady-state bookkeeping (no growth, no trim)
        row4 = row.reshape(1, 1, 1, int(attn.head_dim))
        local.keys[..., write_idx:write_idx + 1, :] = row4
        local.values[..., write_idx:write_idx + 1, :] = row4
        local.offset += 1
        local._idx = write_idx + 1

        self.fused_decode_calls += 1
        out = heads.reshape(1, 1, attn.n_heads * attn.head_dim)
        out = attn._grouped_output_projection(out)
        return attn.wo_b(out)


def _attention_layers(model):
    return getattr(getattr(model, "model", model), "layers", None) or ()


def _patch_deepseek_v4_ratio4_decode_fused_attention(model, *, cache_cls) -> int:
    """Wrap the ratio-4 attention blocks of ``model``; returns how many were wrapped (reference :1792).

    Nothing is installed while the fused decode gate is off. Layers are found under ``model.layers``
    (or ``model.model.layers``); a layer takes part when its ``self_attn`` block has
    ``compress_ratio == 4`` and an indexer. The count is also left on the model.
    """
    if not decode_attention_kernel.fused_decode_enabled():
        object.__setattr__(model, "_moespresso_dsv4_fused_decode_attention_layers", 0)
        return 0
    patched = 0
    for layer in _attention_layers(model):
        attn = getattr(layer, "self_attn", None)
        if attn is None or getattr(attn, "_moespresso_dsv4_fused_decode_attention", False):
            continue
        if int(getattr(attn, "compress_ratio", 0) or 0) != 4 or not hasattr(attn, "indexer"):
            continue
        object.__setattr__(layer, "self_attn", _Ratio4DecodeFusedAttention(attn, cache_cls=cache_cls))
        patched += 1
    object.__setattr__(model, "_moespresso_dsv4_fused_decode_attention_layers", patched)
    return patched


# ---------------------------------------------------------------- ratio-4 prefill fast path

def _dsv4_prefill_pooled_qat(*args) -> torch.Tensor:
    """QAT of pooled indexer rows on the prefill path (reference :752); same kernel as the decode side."""
    return indexer_score_kernel.indexer_qat_rows(_rows_argument(args, "_dsv4_prefill_pooled_qat"))


class _Ratio4PrefillFastAttention:
    """DS4 ratio-4 prefill through the live-layout kernels (reference :1305).

    Projections, norms, rope and cache update run through the wrapped block's own modules and the rope
    seam; the indexer queries take the live QAT, the pool rows the pooled QAT cache, scores come from the
    tiled score kernel, the selection is the deterministic top-k sorted ascending, and attention is the
    indexed mixed prefill consumer on BHLD operands. Single-token calls, other ratios, other cache
    classes and blocks without an indexer go to the wrapped block.
    """

    def __init__(self, original, *, cache_cls):
        self._original = original
        self._cache_cls = cache_cls
        self._moespresso_dsv4_ratio4_prefill_fast_path = True
        self._moespresso_dsv4_ratio4_prefill_fast_calls = 0
        self._moespresso_dsv4_ratio4_prefill_fast_tokens = 0

    def __getattr__(self, name: str):
        return getattr(self._original, name)

    def _attend(self, q, kv, pooled, topk, offset, out_dtype):
        from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

        attn = self._original
        if q.dtype == torch.float16:
            consumer, q_in = iak.indexed_mixed_attention_prefill_live_f16, q
        else:
            consumer, q_in = iak.indexed_mixed_attention_prefill_live_f32, q.to(torch.float32)
        heads = consumer(q_in, kv.to(torch.float16), pooled.to(torch.float16), topk, attn.attn_sink.to(torch.float32),
                         pos0=offset, window=int(attn.args.sliding_window), ratio=int(attn.compress_ratio))
        out = _seam.fused_partial_rope(heads, attn.rope.inv_freq, offset=offset, inverse=True)
        batch, _, tokens, _ = out.shape
        out = out.transpose(1, 2).reshape(batch, tokens, attn.n_heads * attn.head_dim)
        # the consumer and the inverse rope run in float32; the projections take the block's element type
        return attn.wo_b(attn._grouped_output_projection(out.to(out_dtype)))

    def __call__(self, x, mask=None, cache=None):
        from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

        attn = self._original
        batch, tokens, _ = x.shape
        if (int(tokens) <= 1 or int(batch) != 1 or int(getattr(attn, "compress_ratio", 0) or 0) != 4
                or not isinstance(cache, self._cache_cls) or not hasattr(attn, "indexer")):
            return attn(x, mask=mask, cache=cache)

        offset = int(cache.offset)
        q_residual = attn.q_norm(attn.wq_a(x))
        q = attn.wq_b(q_residual).reshape(batch, tokens, attn.n_heads, attn.head_dim)
        q = torch.nn.functional.rms_norm(q, (int(attn.head_dim),), weight=None, eps=float(attn.args.rms_norm_eps))
        q = q.transpose(1, 2)
        kv = attn.kv_norm(attn.wkv(x)).reshape(batch, tokens, 1, attn.head_dim).transpose(1, 2)
        q = _seam.fused_partial_rope(q, attn.rope.inv_freq, offset=offset)
        kv = _seam.fused_partial_rope(kv, attn.rope.inv_freq, offset=offset)
        kv, _ = cache.update_and_fetch(kv, kv)

        pooled = attn.compressor(x, attn.compress_rope, cache, offset)
        n_pool = int(pooled.shape[1])
        if n_pool <= 0:
            topk = torch.zeros((batch, tokens, 0), dtype=torch.int32, device=x.device)
            return self._attend(q, kv, pooled, topk, offset, x.dtype)

        indexer = attn.indexer
        if n_pool <= int(indexer.index_topk):
            row_ids = torch.arange(n_pool, dtype=torch.int32, device=x.device)
            topk = row_ids[None, None, :].expand(batch, tokens, n_pool).contiguous()
        else:
            index_pooled = indexer.compressor(x, attn.compress_rope, cache, offset, state_key="indexer_state")
            q_idx = indexer.wq_b(q_residual).reshape(batch, tokens, indexer.n_heads, indexer.head_dim).transpose(1, 2)
            q_idx = _seam.fused_partial_rope(q_idx, attn.rope.inv_freq, offset=offset)
            q_idx = iak.indexer_q_qat_live(q_idx.to(torch.float32))
            index_pooled_qat, _, _ = pooled_qat_update(getattr(cache, "indexer_state", None), index_pooled)
            weights = indexer.weights_proj(x).to(torch.float32) * (int(indexer.n_heads) ** -0.5) * float(indexer.scale)
            q_scores, comp_scores = iak.indexer_score_operands(q_idx, index_pooled_qat)
            scores = iak.indexer_scores_tiled_live(q_scores, weights, comp_scores, pos0=offset,
                                                   ratio=int(attn.compress_ratio))
            topk_rows = min(int(indexer.index_topk), int(index_pooled_qat.shape[1]))
            topk = indexer_score_kernel.topk_select(scores, topk_rows)
            topk = torch.sort(topk, dim=-1).values.to(torch.int32)

        out = self._attend(q, kv, pooled, topk, offset, x.dtype)
        self._moespresso_dsv4_ratio4_prefill_fast_calls += 1
        self._moespresso_dsv4_ratio4_prefill_fast_tokens += int(tokens)
        return out


def _patch_deepseek_v4_ratio4_prefill_fast_path(model, *, cache_cls) -> int:
    """Install the ratio-4 prefill fast path on the layers of ``model`` (reference :1482)."""
    patched = 0
    for layer in _attention_layers(model):
        attn = getattr(layer, "self_attn", None)
        if attn is None or getattr(attn, "_moespresso_dsv4_ratio4_prefill_fast_path", False):
            continue
        if int(getattr(attn, "compress_ratio", 0) or 0) != 4 or not hasattr(attn, "indexer"):
            continue
        object.__setattr__(layer, "self_attn", _Ratio4PrefillFastAttention(attn, cache_cls=cache_cls))
        patched += 1
    object.__setattr__(model, "_moespresso_dsv4_ratio4_prefill_fast_path_layers", patched)
    return patched
