"""Dispatch of the Qwen/Ornith full-attention layers to the 8-bit-KV attention kernels.

Mirror of the reference module ``src/moespresso/runtime/qwen/full_attention.py``: the same flags,
per-call fail-closed eligibility order, engagement counters and install/statistics helpers
(reference :72-166 flags, :196-276 eligibility, :278-409 forward, :425-470 install/stats), with
``moespresso_amd.runtime.qwen.kquant`` in the place of ``mlx_kquant`` and torch modules in the
place of the MLX ones.

The wrapped ``inner`` module is the model's own attention block. It must expose ``q_proj``,
``k_proj``, ``v_proj``, ``o_proj``, ``q_norm``, ``k_norm``, ``rope(x, offset=...)``, ``scale``,
``num_attention_heads`` and ``num_key_value_heads``, and, for calls this wrapper declines,
``stock_attention(queries, keys, values, cache=..., scale=..., mask=...)`` — the model's composed
attention. This package does not provide a composed fallback of its own: an ineligible call goes to
the model's, and a model without one gets a ``RuntimeError``.
"""

from __future__ import annotations

import os

import torch

from moespresso_amd import _lib
from moespresso_amd.runtime.qwen import kquant as kq

# Family kill switch (reference :72-74); "0" installs nothing.
_QWEN_PREFILL_FLASH_D256 = os.environ.get("MOESPRESSO_QWEN_PREFILL_FLASH_D256", "1") == "1"
# Long-context 8-bit decode route and its merge option (reference :81-87).
_QWEN_DECODE_Q8_TILE16 = os.environ.get("MOESPRESSO_QWEN_DECODE_Q8_TILE16", "1") == "1"
_QWEN_DECODE_Q8_DIMENSION_MERGE = os.environ.get("MOESPRESSO_QWEN_DECODE_Q8_DIMENSION_MERGE", "1") == "1"
_DECODE_Q8_TILE16_MIN_KEYS = 8192

# Stage name -> (stage id, query rows per tile, keys per tile) of the Metal kernel (reference
# :109-117). The HIP kernel picks its own tiling; the values are passed through so that callers
# and tests that read or patch them keep working.
_STAGE_CONFIGS = {
    "f32": (2, 64, 16),
    "f32w32": (2, 32, 16),
}
_STAGE_NAME = os.environ.get("MOESPRESSO_QWEN_PREFILL_FLASH_D256_STAGE", "f32")
if _STAGE_NAME not in _STAGE_CONFIGS:
    _STAGE_NAME = "f32"
_FLASH_STAGE, _FLASH_BQ, _FLASH_BK = _STAGE_CONFIGS[_STAGE_NAME]

# The served geometry the route is fenced for (reference :119-122).
_FLASH_N_Q_HEADS = 16
_FLASH_N_KV_HEADS = 2
_FLASH_HEAD_DIM = 256

_COUNTERS = ("flash_calls", "decode_calls", "decode_dimension_merge_calls", "fallback_prefill_disabled",
             "fallback_no_cache", "fallback_decode", "fallback_cache", "fallback_mask", "fallback_geometry",
             "fallback_dtype", "fallback_kernel")


def flash_prefill_enabled() -> bool:
    """Whether the flash prefill route is enabled for this process."""
    return _QWEN_PREFILL_FLASH_D256


def _kernel_available() -> bool:
    return getattr(kq, "sdpa_fa_prefill_q8", None) is not None and _lib.hip_available()


def _decode_kernel_available() -> bool:
    return getattr(kq, "sdpa_decode_q8", None) is not None and _lib.hip_available()


def _decode_dimension_merge_available() -> bool:
    return bool(getattr(kq, "HAS_SDPA_DECODE_Q8_DIMENSION_PARALLEL_MERGE", False))


def _quantized_cache_class():
    return kq.QuantizedKVCache


def _cache_is_q8_with_past(cache) -> bool:
    qcls = _quantized_cache_class()
    return (qcls is not None and isinstance(cache, qcls) and getattr(cache, "bits", None) == 8
            and getattr(cache, "group_size", None) == 64 and int(getattr(cache, "offset", 0)) >= 1
            and cache.keys is not None)


class FlashPrefillD256Attention(torch.nn.Module):
    """Send eligible prefill and decode calls of one attention block to the 8-bit-KV kernels.

    Everything around the attention itself (projections, norms, rope, cache update, output gate and
    projection) runs through the wrapped block's own modules, so a declined call computes the block's
    stock result.
    """

    def __init__(self, inner):
        super().__init__()
        self.inner = inner
        self.decode_dimension_merge_enabled = _QWEN_DECODE_Q8_DIMENSION_MERGE and _decode_dimension_merge_available()
        for name in _COUNTERS:
            setattr(self, name, 0)

    # ---- eligibility: the first failing branch is the one counted

    def _geometry_ok(self, queries, decode: bool) -> bool:
        return (int(queries.shape[0]) == 1 and int(queries.shape[1]) == _FLASH_N_Q_HEADS
                and (not decode or int(queries.shape[2]) == 1) and int(queries.shape[3]) == _FLASH_HEAD_DIM
                and self.inner.num_key_value_heads == _FLASH_N_KV_HEADS)

    def _flash_eligible(self, queries, cache, mask) -> bool:
        if not _QWEN_PREFILL_FLASH_D256:
            self.fallback_prefill_disabled += 1
        elif int(queries.shape[2]) <= 1:
            self.fallback_decode += 1
        elif not _cache_is_q8_with_past(cache):
            self.fallback_cache += 1
        elif not (isinstance(mask, str) and mask == "causal"):
            self.fallback_mask += 1
        elif not self._geometry_ok(queries, decode=False):
            self.fallback_geometry += 1
        elif queries.dtype != torch.float32:
            self.fallback_dtype += 1
        elif not _kernel_available():
            self.fallback_kernel += 1
        else:
            return True
        return False

    def _decode_eligible(self, queries, cache, mask) -> bool:
        if not _QWEN_DECODE_Q8_TILE16:
            self.fallback_decode += 1
        elif not _cache_is_q8_with_past(cache):
            self.fallback_cache += 1
        elif int(cache.offset) + int(queries.shape[2]) < _DECODE_Q8_TILE16_MIN_KEYS:
            self.fallback_decode += 1
        elif mask is not None:
            self.fallback_mask += 1
        elif not self._geometry_ok(queries, decode=True):
            self.fallback_geometry += 1
        elif queries.dtype != torch.float32:
            self.fallback_dtype += 1
        elif not _decode_kernel_available():
            self.fallback_kernel += 1
        else:
            return True
        return False

    # ---- forward

    def _stock(self, queries, keys, values, cache, mask):
        stock = getattr(self.inner, "stock_attention", None)
        if stock is None:
            raise RuntimeError("call is not eligible for the 8-bit-KV kernels and the wrapped block provides no "
                               "stock_attention to fall back to")
        return stock(queries, keys, values, cache=cache, scale=self.inner.scale, mask=mask)

    def forward(self, x, mask=None, cache=None):
        inner = self.inner
        B, L, _ = x.shape
        heads = inner.num_attention_heads
        kv_heads = inner.num_key_value_heads

        # the query projection carries the output gate in its second half
        queries, gate = inner.q_proj(x).reshape(B, L, heads, -1).chunk(2, dim=-1)
        gate = gate.reshape(B, L, -1)
        queries = inner.q_norm(queries).transpose(1, 2)
        keys = inner.k_norm(inner.k_proj(x).reshape(B, L, kv_heads, -1)).transpose(1, 2)
        values = inner.v_proj(x).reshape(B, L, kv_heads, -1).transpose(1, 2)

        if cache is None:
            self.fallback_no_cache += 1
            output = self._stock(inner.rope(queries), inner.rope(keys), values, None, mask)
        else:
            queries = inner.rope(queries, offset=cache.offset)
            keys = inner.rope(keys, offset=cache.offset)
            if int(queries.shape[2]) == 1:
                if self._decode_eligible(queries, cache, mask):
                    q_keys, q_values = cache.update_and_fetch(keys, values)
                    self.decode_calls += 1
                    options = {}
                    if self.decode_dimension_merge_enabled:
                        self.decode_dimension_merge_calls += 1
                        options["dimension_parallel_merge"] = True
                    output = kq.sdpa_decode_q8(queries.contiguous(), *q_keys, *q_values, inner.scale, group_size=64,
                                               bits=8, splits=128, stage=2, compute=1, tile_c=16, **options)
                else:
                    keys, values = cache.update_and_fetch(keys, values)
                    output = self._stock(queries, keys, values, cache, mask)
            elif self._flash_eligible(queries, cache, mask):
                # the prefix as it stood before this chunk; the update keeps the cache right for later
                # chunks and for decode, its return value is not needed here
                past_k, past_v = cache.state
                # the chunk attends itself through the 8-bit round trip, the values a later read of
                # the cache reconstructs (reference :357-369); taken before the update on purpose
                gs, bits = cache.group_size, cache.bits
                self_k = kq.dequantize(*kq.quantize(keys, group_size=gs, bits=bits), group_size=gs, bits=bits)
                self_v = kq.dequantize(*kq.quantize(values, group_size=gs, bits=bits), group_size=gs, bits=bits)
                cache.update_and_fetch(keys, values)
                self.flash_calls += 1
                output = kq.sdpa_fa_prefill_q8(queries.contiguous(), *past_k, *past_v, self_k, self_v, inner.scale,
                                               bq=_FLASH_BQ, bk=_FLASH_BK, stage=_FLASH_STAGE)
            else:
                keys, values = cache.update_and_fetch(keys, values)
                output = self._stock(queries, keys, values, cache, mask)

        output = output.transpose(1, 2).reshape(B, L, -1)
        return inner.o_proj(output * torch.sigmoid(gate))


def _iter_full_attention_layers(model):
    """Every decoder layer that carries a full-attention block (linear-attention layers are skipped)."""
    layers = None
    for path in (("language_model", "model", "layers"), ("model", "layers"), ("layers",)):
        obj = model
        for attr in path:
            obj = getattr(obj, attr, None)
            if obj is None:
                break
        if obj is not None:
            layers = obj
            break
    if layers is None:
        return
    for layer in layers:
        if getattr(layer, "is_linear", True) or getattr(layer, "self_attn", None) is None:
            continue
        yield layer


def install_flash_prefill_attention(model) -> int:
    """Wrap the full-attention layers; returns how many were wrapped (0 when both routes are off or
    their kernels are missing; already wrapped layers are left alone)."""
    prefill_ready = _QWEN_PREFILL_FLASH_D256 and _kernel_available()
    decode_ready = _QWEN_DECODE_Q8_TILE16 and _decode_kernel_available()
    if not (prefill_ready or decode_ready):
        return 0
    installed = 0
    for layer in _iter_full_attention_layers(model):
        if isinstance(layer.self_attn, FlashPrefillD256Attention):
            continue
        layer.self_attn = FlashPrefillD256Attention(layer.self_attn)
        installed += 1
    return installed


def flash_prefill_attention_stats(model) -> dict:
    """Engagement counters summed over the wrapped layers."""
    stats = {"wrapped_layers": 0}
    stats.update({name: 0 for name in _COUNTERS})
    for layer in _iter_full_attention_layers(model):
        attn = layer.self_attn
        if not isinstance(attn, FlashPrefillD256Attention):
            continue
        stats["wrapped_layers"] += 1
        for name in _COUNTERS:
            stats[name] += int(getattr(attn, name))
    return stats
