"""One-layer DS4 attention speed replay.

Counterpart of the reference's ``src/moespresso/runtime/deepseek_v4/ratio4_attention_replay.py``: time
calls through one ratio-4 attention layer with seeded compressed pools, per replay case (pool rows,
top-k width), optionally with a per-stage breakdown, without running a whole model. The reference
loads a served package and takes one of its layers (:545-575); loading packages is outside this
package, so the layer comes in as an argument, and ``synthetic_attention_block`` builds a stand-in
with random weights and the served head geometry for runs without a model. Everything timed goes
through the same wrappers and kernels a real layer would use.

Speed diagnostic only: it says nothing about output quality.

    python -m moespresso_amd.runtime.deepseek_v4.ratio4_attention_replay --rows 961 7618 --stage-profile
"""

from __future__ import annotations

import argparse
import json
import math
from dataclasses import dataclass
from types import SimpleNamespace
from typing import Any, Callable, Sequence

import torch


@dataclass(frozen=True)
class Ratio4ReplayCase:
    name: str
    pooled_rows: int
    index_topk: int
    cache: bool = True


def default_replay_cases() -> tuple[Ratio4ReplayCase, ...]:
    """The reference's speed-goal cases (:30-44): 961 rows (bounded long prompt), 7618 rows (long
    context), and the splits where the top-k is skipped because the pool is not larger than it."""
    return (
        Ratio4ReplayCase("local_no_compressed_pool", 0, 512, cache=False),
        Ratio4ReplayCase("ratio4_rows961_topk_active", 961, 512),
        Ratio4ReplayCase("ratio4_rows7618_topk_active", 7618, 512),
        Ratio4ReplayCase("ratio4_rows961_topk_skipped", 961, 2000),
        Ratio4ReplayCase("ratio4_rows512_topk_skipped", 512, 512),
    )


def selected_replay_cases(*, include_splits: bool, pooled_rows: Sequence[int] | None = None, index_topk: int = 512,
                          ratio_label: str = "ratio4") -> tuple[Ratio4ReplayCase, ...]:
    """Case selection of the reference (:47-66)."""
    if pooled_rows:
        return tuple(Ratio4ReplayCase(f"{ratio_label}_rows{int(rows)}_topk{int(index_topk)}", int(rows), int(index_topk))
                     for rows in pooled_rows)
    cases = default_replay_cases()
    return cases if include_splits else cases[:3]


def _set_index_topk(attn: Any, topk: int) -> None:
    indexer = getattr(attn, "indexer", None)
    if indexer is None:
        return
    object.__setattr__(indexer, "index_topk", int(topk))
    original = getattr(indexer, "_original", None)
    if original is not None and hasattr(original, "index_topk"):
        object.__setattr__(original, "index_topk", int(topk))


# ---------------------------------------------------------------- stage profile

class _StageProfile:
    """Per-stage device time, from events recorded on the current stream around each stage call."""

    def __init__(self) -> None:
        self._pending: list[tuple[str, torch.cuda.Event, torch.cuda.Event]] = []
        self.rows: dict[str, dict[str, float | int]] = {}

    def reset(self) -> None:
        self._pending.clear()
        self.rows.clear()

    def record(self, name: str, fn: Callable[[], Any]) -> Any:
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        result = fn()
        stop.record()
        self._pending.append((name, start, stop))
        return result

    def collect(self) -> dict[str, dict[str, float | int]]:
        torch.cuda.synchronize()
        for name, start, stop in self._pending:
            row = self.rows.setdefault(name, {"calls": 0, "seconds": 0.0})
            row["calls"] += 1
            row["seconds"] += start.elapsed_time(stop) * 1e-3
        self._pending.clear()
        return self.rows


# module attribute -> stage name; the wrappers look these callables up on their modules at call time,
# so replacing the attribute is enough to time them
_STAGES = (
    ("decode_attention_kernel", "fused_decode_prep", "decode_prep"),
    ("decode_attention_kernel", "fused_decode_sdpa", "decode_sdpa"),
    ("indexer_score_kernel", "indexer_qat_rows", "indexer_qat"),
    ("indexer_score_kernel", "fused_qat_indexer_scores", "indexer_scores"),
    ("indexer_score_kernel", "topk_select", "topk"),
    ("attention_seam_kernel", "fused_partial_rope", "partial_rope"),
    ("indexed_attention_kernel", "indexer_q_qat_live", "prefill_q_qat"),
    ("indexed_attention_kernel", "indexer_scores_tiled_live", "prefill_scores"),
    ("indexed_attention_kernel", "indexed_mixed_attention_prefill_live_f16", "prefill_attention"),
    ("indexed_attention_kernel", "indexed_mixed_attention_prefill_live_f32", "prefill_attention"),
)


class _StagePatch:
    """Route the stage callables through a ``_StageProfile`` for the duration of a ``with`` block."""

    def __init__(self, profile: _StageProfile):
        self._profile = profile
        self._saved: list[tuple[Any, str, Any]] = []

    def __enter__(self):
        import importlib

        for module_name, attr, stage in _STAGES:
            module = importlib.import_module(f"moespresso_amd.runtime.deepseek_v4.{module_name}")
            original = getattr(module, attr)
            self._saved.append((module, attr, original))

            def timed(*args, _fn=original, _stage=stage, **kwargs):
                return self._profile.record(_stage, lambda: _fn(*args, **kwargs))

            setattr(module, attr, timed)
        return self._profile

    def __exit__(self, *exc):
        for module, attr, original in reversed(self._saved):
            setattr(module, attr, original)
        self._saved.clear()
        return False


# ---------------------------------------------------------------- stand-in layer for runs without a model

def rope_inverse_frequencies(dim: int, base: float, yarn: dict | None = None) -> torch.Tensor:
    """Float32 rope inverse frequencies with the YaRN ramp folded in (reference attention.py:71-102)."""
    idx = torch.arange(0, dim, 2, dtype=torch.float64)
    freqs = 1.0 / (float(base) ** (idx / dim))
    if yarn:
        factor, original = float(yarn["factor"]), float(yarn["original_seq_len"])
        beta_fast, beta_slow = float(yarn.get("beta_fast", 32.0)), float(yarn.get("beta_slow", 1.0))
        if factor > 1.0 and original > 0:
            def correction_dim(n: float) -> float:
                return dim * math.log(original / (n * 2.0 * math.pi)) / (2.0 * math.log(base))

            low = max(math.floor(correction_dim(beta_fast)), 0)
            high = min(math.ceil(correction_dim(beta_slow)), dim - 1)
            if low == high:
                high += 0.001
            ramp = (torch.arange(dim // 2, dtype=torch.float64) - low) / (high - low)
            smooth = 1.0 - ramp.clamp(0.0, 1.0)
            freqs = freqs / factor * (1.0 - smooth) + freqs * smooth
    return freqs.to(torch.float32)


class SyntheticRing:
    """The rotating local cache in its steady state: a full ring of ``max_size`` rows."""

    def __init__(self, keys: torch.Tensor, offset: int, idx: int):
        self.keys, self.values = keys, keys.clone()
        self.offset, self._idx = int(offset), int(idx)
        self.max_size, self.keep = int(keys.shape[2]), 0


class SyntheticCache:
    """Fields of the DS4 cache the wrappers read: the ring, the two pool states, offset, update, trim."""

    def __init__(self, ring: SyntheticRing):
        self.local = ring
        self.compressor_state: dict = {}
        self.indexer_state: dict = {}

    @property
    def offset(self) -> int:
        return self.local.offset

    def update_and_fetch(self, keys, values):
        return keys, values

    def trim(self, n):
        return n


class _PoolCompressor:
    """Hands back the pool the cache state holds (a steady-state token appends no pool row)."""

    def __call__(self, x, rope, cache, offset, state_key="compressor_state"):
        return getattr(cache, state_key)["pooled"]


def synthetic_attention_block(device, *, hidden: int = 4096, n_heads: int = 64, q_lora: int = 1024,
                              index_heads: int = 64, index_topk: int = 512, sliding_window: int = 128,
                              seed: int = 0) -> Any:
    """A ratio-4 attention block with random float16 weights and the served head geometry."""
    gen = torch.Generator().manual_seed(seed)

    def linear(n_in, n_out):
        lin = torch.nn.Linear(n_in, n_out, bias=False, device=device, dtype=torch.float16)
        with torch.no_grad():
            lin.weight.copy_((torch.randn((n_out, n_in), generator=gen) * n_in ** -0.5).to(torch.float16))
        return lin

    yarn = {"factor": 16.0, "original_seq_len": 65536, "beta_fast": 32, "beta_slow": 1}
    block = SimpleNamespace()
    block.args = SimpleNamespace(sliding_window=sliding_window, rms_norm_eps=1e-6, hidden_size=hidden)
    block.compress_ratio, block.head_dim, block.n_heads = 4, 512, n_heads
    block.rope = SimpleNamespace(dims=64, inv_freq=rope_inverse_frequencies(64, 10000.0).to(device))
    block.compress_rope = SimpleNamespace(dims=64, inv_freq=rope_inverse_frequencies(64, 160000.0, yarn).to(device))
    block.wq_a, block.wq_b = linear(hidden, q_lora), linear(q_lora, n_heads * 512)
    block.q_norm = torch.nn.RMSNorm(q_lora, eps=1e-6, device=device, dtype=torch.float16)
    block.wkv = linear(hidden, 512)
    block.kv_norm = torch.nn.RMSNorm(512, eps=1e-6, device=device, dtype=torch.float16)
    block.compressor = _PoolCompressor()
    block.indexer = SimpleNamespace(n_heads=index_heads, head_dim=128, index_topk=index_topk, scale=128 ** -0.5,
                                    compressor=_PoolCompressor(), wq_b=linear(q_lora, index_heads * 128),
                                    weights_proj=linear(hidden, index_heads))
    block.attn_sink = (torch.randn((n_heads,), generator=gen) * 0.3).to(device)
    block.softmax_scale = 512 ** -0.5
    block.wo_b = linear(n_heads * 512, hidden)
    block._grouped_output_projection = lambda out: out
    return block


def make_seeded_cache(device, *, sliding_window: int, pooled_rows: int, head_dim: int = 512, index_head_dim: int = 128,
                      offset: int = 30000, prime_indexer_qat: bool = True, seed: int = 1) -> SyntheticCache:
    """A steady-state cache with ``pooled_rows`` seeded pool rows (reference :79-109)."""
    from moespresso_amd.runtime.deepseek_v4 import model as dsm

    gen = torch.Generator().manual_seed(seed)
    keys = (torch.randn((1, 1, sliding_window, head_dim), generator=gen) * 0.1).to(torch.float16).to(device)
    cache = SyntheticCache(SyntheticRing(keys, offset, offset % sliding_window))
    if pooled_rows > 0:
        cache.compressor_state["pooled"] = (torch.randn((1, pooled_rows, head_dim), generator=gen) * 0.1).to(
            torch.float16).to(device)
        pool = torch.randn((1, pooled_rows, index_head_dim), generator=gen).to(torch.float16).to(device)
        cache.indexer_state["pooled"] = pool
        if prime_indexer_qat:
            cache.indexer_state["pooled_qat"] = dsm._dsv4_indexer_qat(pool)
            cache.indexer_state["pooled_qat_rows"] = pooled_rows
    return dsm._cache_with_fp8_kv_roundtrip(cache)


# ---------------------------------------------------------------- replay

def _time_case(layer: Callable[..., Any], caches: list, x: torch.Tensor, case: Ratio4ReplayCase, *, repeats: int,
               warmup: int, profile: _StageProfile | None) -> dict[str, Any]:
    """``caches`` holds one fresh cache per call (warm-ups first): the ring append and the pool caches
    start equal every time, and building them is not part of any timing."""
    mask = "causal" if int(x.shape[1]) > 1 else None
    caches = list(caches)
    for _ in range(max(warmup, 0)):
        layer(x, mask=mask, cache=caches.pop(0))
    torch.cuda.synchronize()
    if profile is not None:
        profile.reset()
    seconds = []
    for _ in range(repeats):
        cache = caches.pop(0)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        layer(x, mask=mask, cache=cache)
        stop.record()
        torch.cuda.synchronize()
        seconds.append(start.elapsed_time(stop) * 1e-3)
    seconds.sort()
    row: dict[str, Any] = {"name": case.name, "pooled_rows": case.pooled_rows, "index_topk": case.index_topk,
                           "median_seconds": seconds[len(seconds) // 2], "min_seconds": seconds[0],
                           "repeats": repeats}
    if profile is not None:
        stages = profile.collect()
        row["stages"] = {name: {"calls_per_layer_call": r["calls"] / repeats, "seconds_per_layer_call": r["seconds"] / repeats}
                         for name, r in sorted(stages.items())}
    return row


def run_ratio4_attention_replay(attn: Any, *, cache_cls: type, make_cache: Callable[[Ratio4ReplayCase], Any],
                                hidden_size: int, device, repeats: int = 5, warmup: int = 1,
                                include_splits: bool = False, pooled_rows: Sequence[int] | None = None,
                                index_topk: int = 512, stage_profile: bool = False, input_tokens: int = 1,
                                seed: int = 0) -> dict[str, Any]:
    """Time ``attn`` through the fused decode wrapper (one token) or the prefill fast path (several).

    ``attn`` is a ratio-4 attention block (the wrappers' contract), ``make_cache(case)`` returns a
    fresh cache of class ``cache_cls`` seeded for the case (``None`` for a case without a cache).
    """
    from moespresso_amd.runtime.deepseek_v4 import decode_attention_kernel, indexer_score_kernel
    from moespresso_amd.runtime.deepseek_v4 import model as dsm

    tokens = int(input_tokens)
    if tokens <= 0:
        raise ValueError("input_tokens must be positive")
    compress_ratio = int(getattr(attn, "compress_ratio", 0) or 0)
    cases = selected_replay_cases(include_splits=include_splits, pooled_rows=pooled_rows, index_topk=index_topk,
                                  ratio_label=f"ratio{compress_ratio}")
    if tokens == 1:
        layer = dsm._Ratio4DecodeFusedAttention(attn, cache_cls=cache_cls)
    else:
        layer = dsm._Ratio4PrefillFastAttention(attn, cache_cls=cache_cls)
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn((1, tokens, int(hidden_size)), generator=gen) * 0.05).to(torch.float16).to(device)
    profile = _StageProfile() if stage_profile else None
    gates = (decode_attention_kernel._ENABLED, indexer_score_kernel._ENABLED)
    decode_attention_kernel._ENABLED = indexer_score_kernel._ENABLED = True
    results = []
    try:
        for case in cases:
            if not case.cache or (tokens == 1 and case.pooled_rows <= case.index_topk):
                # without a pool larger than the selection the fused decode contract does not engage and the
                # call belongs to the model's composed path, which this package does not have
                results.append({"name": case.name, "pooled_rows": case.pooled_rows, "index_topk": case.index_topk,
                                "skipped": "served by the wrapped block's composed path"})
                continue
            _set_index_topk(attn, case.index_topk)
            caches = [make_cache(case) for _ in range(max(warmup, 0) + repeats)]
            torch.cuda.synchronize()
            if profile is not None:
                with _StagePatch(profile):
                    results.append(_time_case(layer, caches, x, case, repeats=repeats, warmup=warmup, profile=profile))
            else:
                results.append(_time_case(layer, caches, x, case, repeats=repeats, warmup=warmup, profile=None))
    finally:
        decode_attention_kernel._ENABLED, indexer_score_kernel._ENABLED = gates
    return {
        "metric": "ds4_attention_one_layer_replay",
        "units": "seconds per call through one DS4 ratio-4 attention layer",
        "compress_ratio": compress_ratio,
        "stage_profile": bool(stage_profile),
        "input_tokens": tokens,
        "fused_decode_calls": int(getattr(layer, "fused_decode_calls", 0)),
        "prefill_fast_calls": int(getattr(layer, "_moespresso_dsv4_ratio4_prefill_fast_calls", 0)),
        "quality_note": "speed diagnostic only",
        "cases": results,
    }


def main(argv: Sequence[str] | None = None) -> int:
    parser = argparse.ArgumentParser(
        prog="moespresso-amd-ds4-ratio4-attention-replay",
        description="Time one DS4 ratio-4 attention layer (random weights, served geometry) with seeded compressed pools.")
    parser.add_argument("--repeats", type=int, default=5)
    parser.add_argument("--warmup", type=int, default=1)
    parser.add_argument("--include-splits", action="store_true", help="also run the top-k skipped split cases")
    parser.add_argument("--rows", type=int, nargs="*", default=None, help="pool row counts to replay instead of the defaults")
    parser.add_argument("--index-topk", type=int, default=512)
    parser.add_argument("--input-tokens", type=int, default=1, help="1 = decode token, more = prefill chunk")
    parser.add_argument("--stage-profile", action="store_true")
    parser.add_argument("--hidden-size", type=int, default=4096)
    args = parser.parse_args(argv)
    device = torch.device("cuda:0")
    attn = synthetic_attention_block(device, hidden=args.hidden_size, index_topk=args.index_topk)
    window = int(attn.args.sliding_window)

    def make_cache(case: Ratio4ReplayCase):
        offset = 0 if args.input_tokens > 1 else 30000
        return make_seeded_cache(device, sliding_window=window, pooled_rows=case.pooled_rows, offset=offset)

    report = run_ratio4_attention_replay(attn, cache_cls=SyntheticCache, make_cache=make_cache,
                                         hidden_size=args.hidden_size, device=device, repeats=args.repeats,
                                         warmup=args.warmup, include_splits=args.include_splits, pooled_rows=args.rows,
                                         index_topk=args.index_topk, stage_profile=args.stage_profile,
                                         input_tokens=args.input_tokens)
    print(json.dumps(report, indent=2))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
