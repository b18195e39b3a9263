"""GPU tests of the DS4 layer glue: cache write path, pooled-row QAT cache, decode score contract and
the fused ratio-4 decode attention wrapper, against the NumPy oracle of the two fused kernels.

The cases follow the reference's wrapper tests (tests/test_deepseek_v4_decode_attention_kernel.py
:184-212, :459-578); the composed layer they compare against needs third-party packages, so the oracle
of the fused pair (pinned elsewhere) stands in for it, fed with the projections the wrapper itself saw.
"""

import numpy as np
import pytest
import torch

from moespresso_amd.runtime.deepseek_v4 import decode_attention_kernel as dak
from moespresso_amd.runtime.deepseek_v4 import indexer_score_kernel as isk
from moespresso_amd.runtime.deepseek_v4 import model as dsm
from oracle import ds4
from ds4_standins import OFFSET, Attention, Cache, OtherCache, steady_cache

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _np(t):
    return t.detach().float().cpu().numpy()


def _run_fused(monkeypatch, *, rows=96, idx=37):
    monkeypatch.setattr(dak, "_ENABLED", True)
    attn = Attention(DEV)
    wrapper = dsm._Ratio4DecodeFusedAttention(attn, cache_cls=Cache)
    cache = dsm._cache_with_fp8_kv_roundtrip(steady_cache(DEV, rows=rows, idx=idx))
    x = (torch.randn((1, 1, 256), generator=torch.Generator().manual_seed(5)) * 0.05).to(torch.float16).to(DEV)
    seen = {}
    real_prep, real_sdpa = dak.fused_decode_prep, dak.fused_decode_sdpa

    def prep(*a, **k):
        seen["prep_in"] = (a, k)
        seen["prep_out"] = real_prep(*a, **k)
        return seen["prep_out"]

    def sdpa(*a, **k):
        seen["sdpa_in"] = (tuple(t.clone() for t in a), k)  # the window is a view of the ring, appended to later
        return real_sdpa(*a, **k)

    monkeypatch.setattr(dak, "fused_decode_prep", prep)
    monkeypatch.setattr(dak, "fused_decode_sdpa", sdpa)
    window_before = cache.local.keys.clone()
    out = wrapper(x, mask=None, cache=cache)
    torch.cuda.synchronize()
    return attn, wrapper, cache, x, out, seen, window_before


def test_fused_decode_wrapper_matches_oracle_of_the_fused_pair(monkeypatch):
    attn, wrapper, cache, x, out, seen, window_before = _run_fused(monkeypatch)
    assert wrapper.fused_decode_calls == 1 and wrapper.fused_decode_composed_tail_calls == 0
    assert attn.stock_calls == [] and attn.tail_calls == []
    # both compressors advanced once, the indexer one on its own state
    assert attn.compressor.calls == ["compressor_state"] and attn.indexer.compressor.calls == ["indexer_state"]

    (q_idx, pooled_qat, weights, kv_row, inv, params), kw = seen["prep_in"]
    assert kw == {"scale": 128 ** -0.5, "topk": 64}
    assert params.cpu().tolist() == [OFFSET, 37]
    sel, row, scores = seen["prep_out"]
    # the pooled QAT rows are the kernel's QAT of the indexer pool, kept in the cache state
    np.testing.assert_array_equal(_np(pooled_qat), ds4.indexer_qat(_np(cache.indexer_state["pooled"][0])))
    assert cache.indexer_state["pooled_qat_rows"] == 96
    # prepared row and selection against the oracle (selection on the device's own scores)
    o_sel, o_row, o_scores = ds4.fused_decode_prep(_np(q_idx), _np(pooled_qat), _np(weights), _np(kv_row), _np(inv),
                                                   params.cpu().numpy(), scale=128 ** -0.5, topk=64)
    np.testing.assert_array_equal(_np(row).astype(np.float16).view(np.uint16), o_row.astype(np.float16).view(np.uint16))
    np.testing.assert_allclose(_np(scores), o_scores, rtol=2e-5, atol=2e-5)
    np.testing.assert_array_equal(sel.cpu().numpy(), ds4.radix_select_topk(_np(scores), 64))

    (q, window, row_in, pooled, sel_in, sinks, inv2, params2), kw2 = seen["sdpa_in"]
    np.testing.assert_array_equal(_np(window), _np(window_before[0, 0]))  # the ring as it stood before the append
    want = ds4.fused_decode_sdpa(_np(q), _np(window), _np(row_in), _np(pooled), sel_in.cpu().numpy(), _np(sinks),
                                 _np(inv2), params2.cpu().numpy(), scale=512 ** -0.5).astype(np.float32)
    got = _np(attn.heads_seen).reshape(8, 512)
    assert np.abs(got - want).max() < 2e-3
    np.testing.assert_array_equal(_np(out), _np(attn.wo_b(attn.heads_seen)))

    # direct append: ring slot 37 holds the prepared row in keys and values, counters moved by one
    assert cache.local.offset == OFFSET + 1 and cache.local._idx == 38
    np.testing.assert_array_equal(_np(cache.local.keys[0, 0, 37]), _np(row))
    np.testing.assert_array_equal(_np(cache.local.values[0, 0, 37]), _np(row))
    untouched = [i for i in range(128) if i != 37]
    np.testing.assert_array_equal(_np(cache.local.keys[0, 0, untouched]), _np(window_before[0, 0, untouched]))
    assert cache.update_calls == 0  # the rounded append bypasses update_and_fetch


def test_fused_decode_wrapper_wraps_the_ring_write_slot(monkeypatch):
    attn, wrapper, cache, x, out, seen, _ = _run_fused(monkeypatch, idx=128)
    (_, _, _, _, _, params), _ = seen["prep_in"]
    assert params.cpu().tolist() == [OFFSET, 0]
    assert cache.local._idx == 1
    np.testing.assert_array_equal(_np(cache.local.keys[0, 0, 0]), _np(seen["prep_out"][1]))


def test_fused_decode_wrapper_hands_short_pools_to_the_composed_tail(monkeypatch):
    attn, wrapper, cache, x, out, seen, window_before = _run_fused(monkeypatch, rows=32)
    assert wrapper.fused_decode_calls == 0 and wrapper.fused_decode_composed_tail_calls == 1
    assert "prep_in" not in seen
    (kw,) = attn.tail_calls
    assert kw["run_indexer"] is True and kw["topk"] is None and kw["offset"] == OFFSET
    assert tuple(kw["q"].shape) == (1, 1, 8, 512) and tuple(kw["kv"].shape) == (1, 1, 1, 512)
    # nothing was appended by the wrapper itself
    np.testing.assert_array_equal(_np(cache.local.keys), _np(window_before))
    assert cache.local.offset == OFFSET


def test_fused_decode_wrapper_without_a_tail_fails_loudly(monkeypatch):
    monkeypatch.setattr(dak, "_ENABLED", True)
    attn = Attention(DEV)
    attn.composed_decode_tail = None
    wrapper = dsm._Ratio4DecodeFusedAttention(attn, cache_cls=Cache)
    cache = dsm._cache_with_fp8_kv_roundtrip(steady_cache(DEV, rows=32))
    x = torch.zeros((1, 1, 256), dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="composed_decode_tail"):
        wrapper(x, mask=None, cache=cache)


def test_fused_decode_wrapper_delegates_outside_contract(monkeypatch):
    attn = Attention(DEV)
    wrapper = dsm._Ratio4DecodeFusedAttention(attn, cache_cls=Cache)
    x = torch.zeros((1, 1, 256), dtype=torch.float16, device=DEV)
    cache = steady_cache(DEV, rows=96)
    monkeypatch.setattr(dak, "_ENABLED", False)                      # gate off
    wrapper(x, mask=None, cache=dsm._cache_with_fp8_kv_roundtrip(steady_cache(DEV, rows=96)))
    monkeypatch.setattr(dak, "_ENABLED", True)
    wrapper(x, mask=None, cache=cache)                               # no rounded-append contract on the cache
    marked = dsm._cache_with_fp8_kv_roundtrip(steady_cache(DEV, rows=96))
    wrapper(torch.zeros((1, 4, 256), dtype=torch.float16, device=DEV), mask=None, cache=marked)  # prefill shape
    wrapper(x.float(), mask=None, cache=marked)                      # element type
    wrapper(x, mask=None, cache=dsm._cache_with_fp8_kv_roundtrip(steady_cache(DEV, rows=96, cls=OtherCache)))
    cold = dsm._cache_with_fp8_kv_roundtrip(steady_cache(DEV, rows=96, offset=100))
    wrapper(x, mask=None, cache=cold)                                # ring not yet full
    wrapper(x, mask=None, cache=None)
    assert len(attn.stock_calls) == 7
    assert wrapper.fused_decode_calls == 0 and attn.compressor.calls == []


def test_patch_installs_fused_decode_wrapper_by_gate(monkeypatch):
    from types import SimpleNamespace
    layers = [SimpleNamespace(self_attn=Attention(DEV)), SimpleNamespace(self_attn=SimpleNamespace(compress_ratio=128)),
              SimpleNamespace()]
    model = SimpleNamespace(model=SimpleNamespace(layers=layers))
    monkeypatch.setattr(dak, "_ENABLED", False)
    assert dsm._patch_deepseek_v4_ratio4_decode_fused_attention(model, cache_cls=Cache) == 0
    monkeypatch.setattr(dak, "_ENABLED", True)
    assert dsm._patch_deepseek_v4_ratio4_decode_fused_attention(model, cache_cls=Cache) == 1
    assert isinstance(layers[0].self_attn, dsm._Ratio4DecodeFusedAttention)
    assert model._moespresso_dsv4_fused_decode_attention_layers == 1
    assert dsm._patch_deepseek_v4_ratio4_decode_fused_attention(model, cache_cls=Cache) == 0  # idempotent
    assert layers[0].self_attn.n_heads == 8  # attributes of the wrapped block stay reachable


def test_fp8_cache_write_path_rounds_rows_once(monkeypatch):
    cache = steady_cache(DEV, rows=8)
    wrapped = dsm._cache_with_fp8_kv_roundtrip(cache)
    assert wrapped is cache and cache._moespresso_dsv4_fp8_kv_cache
    assert dsm._cache_with_fp8_kv_roundtrip(cache) is cache  # idempotent: still one layer of rounding
    rng = np.random.default_rng(3)
    rows = torch.from_numpy(rng.standard_normal((1, 1, 5, 512), dtype=np.float32)).to(DEV)
    k, v = cache.update_and_fetch(rows, rows)
    assert cache.update_calls == 1 and k is v
    np.testing.assert_array_equal(_np(k), ds4.fp8_kv_roundtrip(_np(rows)))
    k2, v2 = cache.update_and_fetch(rows, rows.clone())
    np.testing.assert_array_equal(_np(v2), _np(k2))
    # 16-bit rows: float32 arithmetic, cast back
    half = rows.to(torch.float16)
    kh, _ = cache.update_and_fetch(half, half)
    assert kh.dtype == torch.float16
    np.testing.assert_array_equal(_np(kh), ds4.fp8_kv_roundtrip(_np(half)).astype(np.float16).astype(np.float32))
    # rows of another width and empty tensors pass through
    odd = torch.zeros((1, 1, 2, 128), device=DEV)
    assert dsm._deepseek_v4_fp8_kv_roundtrip(odd) is odd
    with pytest.raises(dsm.DeepseekV4RuntimeLoadError):
        dsm._deepseek_v4_fp8_kv_roundtrip(torch.zeros((2, 96), device=DEV), head_dim=96, rot_dim=64)


def test_trim_clears_the_derived_pool_caches():
    cache = dsm._cache_with_compressed_pool_aux_trim_clear(steady_cache(DEV, rows=8))
    cache.indexer_state.update(pooled_qat=1, pooled_qat_rows=8)
    cache.compressor_state.update(pooled_fp8=1, pooled_fp8_rows=8)
    assert cache.trim(3) == 3 and cache.trim_calls == 1
    assert "pooled_qat" not in cache.indexer_state and "pooled_qat_rows" not in cache.indexer_state
    assert "pooled_fp8" not in cache.compressor_state and "pooled" in cache.compressor_state


def test_pooled_qat_update_is_incremental_and_bit_equal_to_a_full_pass():
    rng = np.random.default_rng(8)
    pool = torch.from_numpy(rng.standard_normal((1, 40, 128), dtype=np.float32)).to(torch.float16).to(DEV)
    state = {}
    a, cached, new = dsm.pooled_qat_update(state, pool[:, :24])
    assert (cached, new) == (0, 24) and state["pooled_qat_rows"] == 24
    b, cached, new = dsm.pooled_qat_update(state, pool[:, :24])
    assert (cached, new) == (24, 0) and b is a
    c, cached, new = dsm.pooled_qat_update(state, pool)
    assert (cached, new) == (24, 16) and state["pooled_qat_rows"] == 40
    np.testing.assert_array_equal(_np(c), _np(dsm._dsv4_indexer_qat(pool)))
    np.testing.assert_array_equal(_np(c), ds4.indexer_qat(_np(pool)))
    # a cache longer than the pool (after a trim) is not trusted
    d, cached, new = dsm.pooled_qat_update({"pooled_qat": c, "pooled_qat_rows": 40}, pool[:, :10])
    assert (cached, new) == (0, 10) and tuple(d.shape) == (1, 10, 128)
    # without a state dict nothing is kept
    e, cached, new = dsm.pooled_qat_update(None, pool[:, :3])
    assert (cached, new) == (0, 3)


def test_decode_score_contract_selects_on_the_fused_score_row(monkeypatch):
    monkeypatch.setattr(isk, "_ENABLED", True)
    attn = Attention(DEV, index_heads=64, topk=16)
    contract = dsm._IndexerDS4ScoreContract(attn.indexer, 4, layer_index=0)
    cache = steady_cache(DEV, rows=200)
    x = (torch.randn((1, 1, 256), generator=torch.Generator().manual_seed(2)) * 0.05).to(torch.float16).to(DEV)
    q_res = attn.q_norm(attn.wq_a(x))
    topk = contract(x, q_res, attn.compress_rope, attn.rope, cache, OFFSET)
    assert tuple(topk.shape) == (1, 1, 16) and topk.dtype == torch.int32
    # the same row through the kernels by hand
    q = attn.indexer.wq_b(q_res).reshape(1, 1, 64, 128).transpose(1, 2)
    from moespresso_amd.runtime.deepseek_v4 import attention_seam_kernel as seam
    q = seam.fused_partial_rope(q, attn.rope.inv_freq, offset=OFFSET)
    w = attn.indexer.weights_proj(x).float() * 64 ** -0.5
    scores = isk.fused_qat_indexer_scores(q, cache.indexer_state["pooled_qat"], w, 128 ** -0.5)
    np.testing.assert_array_equal(topk.cpu().numpy().reshape(-1), ds4.radix_select_topk(_np(scores), 16))
    o_scores = ds4.fused_qat_indexer_scores(_np(q), _np(cache.indexer_state["pooled_qat"]), _np(w), 128 ** -0.5)
    np.testing.assert_allclose(_np(scores), o_scores.reshape(-1), rtol=2e-5, atol=2e-5)
    c = "_moespresso_dsv4_indexer_score_contract_"
    assert getattr(contract, c + "calls") == 1 and getattr(contract, c + "fused_score_calls") == 1
    assert getattr(contract, c + "new_qat_pooled_rows") == 200 and getattr(contract, c + "topk_rows") == 16
    # second token: the pool rows are reused
    contract(x, q_res, attn.compress_rope, attn.rope, cache, OFFSET + 1)
    assert getattr(contract, c + "cached_pooled_rows") == 200 and getattr(contract, c + "new_qat_pooled_rows") == 200
    # every token so far advanced the stateful compressor exactly once
    assert attn.indexer.compressor.positions == [OFFSET, OFFSET + 1] and cache.indexer_state["advances"] == 2
    # prefill shapes go to the wrapped indexer, and so does a decode token while the score gate is off:
    # both before the compressor is touched, so the wrapped indexer's own advance is the only one
    contract(torch.zeros((1, 4, 256), dtype=torch.float16, device=DEV), q_res, None, None, cache, 0)
    assert attn.indexer.stock_calls == 1 and cache.indexer_state["advances"] == 3
    monkeypatch.setattr(isk, "_ENABLED", False)
    assert contract(x, q_res, attn.compress_rope, attn.rope, cache, OFFSET + 2) is None
    assert attn.indexer.stock_calls == 2
    assert attn.indexer.compressor.positions == [OFFSET, OFFSET + 1, 0, OFFSET + 2]
    assert cache.indexer_state["advances"] == 4      # one advance per token, gate on or off
    fused_before = getattr(contract, c + "fused_score_calls")
    # once engaged the call finishes here even when the pool rows arrive in another float type
    monkeypatch.setattr(isk, "_ENABLED", True)
    cache.indexer_state.pop("pooled_qat"), cache.indexer_state.pop("pooled_qat_rows")
    monkeypatch.setattr(dsm, "_dsv4_indexer_qat", lambda rows: isk.indexer_qat_rows(rows).to(torch.float16))
    again = contract(x, q_res, attn.compress_rope, attn.rope, cache, OFFSET + 3)
    assert tuple(again.shape) == (1, 1, 16) and attn.indexer.stock_calls == 2
    assert getattr(contract, c + "fused_score_calls") == fused_before + 1 and cache.indexer_state["advances"] == 5


def _prefill_setup(tokens, rows, *, topk, q_dtype=torch.float16):
    attn = Attention(DEV, topk=topk, index_heads=64)
    wrapper = dsm._Ratio4PrefillFastAttention(attn, cache_cls=Cache)
    cache = steady_cache(DEV, rows=rows, offset=0)
    x = (torch.randn((1, tokens, 256), generator=torch.Generator().manual_seed(9)) * 0.05).to(torch.float16).to(DEV)
    return attn, wrapper, cache, x


@pytest.mark.parametrize("rows,topk", [(40, 64), (40, 16)])
def test_prefill_fast_path_matches_oracle_of_the_consumer(rows, topk):
    # 160 tokens from position 0: pool rows (q+1)//4 become visible as the chunk proceeds
    from moespresso_amd.runtime.deepseek_v4 import attention_seam_kernel as seam
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak
    tokens = 160
    attn, wrapper, cache, x = _prefill_setup(tokens, rows, topk=topk)
    out = wrapper(x, mask=None, cache=cache)
    torch.cuda.synchronize()
    assert wrapper._moespresso_dsv4_ratio4_prefill_fast_calls == 1
    assert wrapper._moespresso_dsv4_ratio4_prefill_fast_tokens == tokens
    assert cache.update_calls == 1 and attn.stock_calls == []

    # the same chunk by hand up to the consumer, then the oracle of the consumer
    q_res = attn.q_norm(attn.wq_a(x))
    q = attn.wq_b(q_res).reshape(1, tokens, 8, 512)
    q = torch.nn.functional.rms_norm(q, (512,), eps=1e-6).transpose(1, 2)
    kv = attn.kv_norm(attn.wkv(x)).reshape(1, tokens, 1, 512).transpose(1, 2)
    q = seam.fused_partial_rope(q, attn.rope.inv_freq, offset=0)
    kv = seam.fused_partial_rope(kv, attn.rope.inv_freq, offset=0)
    np.testing.assert_array_equal(_np(cache.last_update[0]), _np(kv))
    pooled = cache.compressor_state["pooled"]
    if rows <= topk:
        ids = np.broadcast_to(np.arange(rows, dtype=np.int32), (tokens, rows))
        assert attn.indexer.compressor.calls == []
    else:
        q_idx = attn.indexer.wq_b(q_res).reshape(1, tokens, 64, 128).transpose(1, 2)
        q_idx = iak.indexer_q_qat_live(seam.fused_partial_rope(q_idx, attn.rope.inv_freq, offset=0).float())
        w = attn.indexer.weights_proj(x).float() * 64 ** -0.5 * 128 ** -0.5
        scores = iak.indexer_scores_tiled_live(q_idx, w, cache.indexer_state["pooled_qat"], pos0=0, ratio=4)
        ids = np.stack([np.sort(ds4.radix_select_topk(_np(scores)[0, t], topk)) for t in range(tokens)]).astype(np.int32)
        assert cache.indexer_state["pooled_qat_rows"] == rows
    want = ds4.indexed_mixed_attention_prefill(_np(q)[0].transpose(1, 0, 2), _np(kv)[0, 0], _np(pooled)[0], ids,
                                               _np(attn.attn_sink), pos0=0, window=128, ratio=4)       # [T, H, 512]
    want_rot = ds4.fused_partial_rope(want.transpose(1, 0, 2).astype(np.float32), _np(attn.rope.inv_freq), offset=0,
                                      inverse=True)                                                     # [H, T, 512]
    heads = _np(attn.heads_seen).reshape(tokens, 8, 512).transpose(1, 0, 2)
    assert attn.heads_seen.dtype == torch.float16
    assert np.abs(heads - want_rot).max() < 2e-3
    np.testing.assert_array_equal(_np(out), _np(attn.wo_b(attn.heads_seen)))


def test_prefill_fast_path_delegates_outside_its_shapes():
    attn, wrapper, cache, x = _prefill_setup(8, 40, topk=16)
    wrapper(x[:, :1], mask=None, cache=cache)                                   # one token
    wrapper(torch.cat([x, x]), mask=None, cache=cache)                          # batch 2
    wrapper(x, mask=None, cache=steady_cache(DEV, rows=40, cls=OtherCache))     # another cache class
    wrapper(x, mask=None, cache=None)
    attn.compress_ratio = 128
    wrapper(x, mask=None, cache=cache)
    assert len(attn.stock_calls) == 5 and wrapper._moespresso_dsv4_ratio4_prefill_fast_calls == 0
    assert cache.update_calls == 0
    from types import SimpleNamespace
    model = SimpleNamespace(layers=[SimpleNamespace(self_attn=Attention(DEV)), SimpleNamespace(self_attn=None)])
    assert dsm._patch_deepseek_v4_ratio4_prefill_fast_path(model, cache_cls=Cache) == 1
    assert dsm._patch_deepseek_v4_ratio4_prefill_fast_path(model, cache_cls=Cache) == 0
    assert model._moespresso_dsv4_ratio4_prefill_fast_path_layers == 0


def test_one_layer_replay_reports_cases_and_stages():
    from moespresso_amd.runtime.deepseek_v4 import ratio4_attention_replay as replay

    attn = replay.synthetic_attention_block(DEV, hidden=256, n_heads=8, q_lora=64, index_heads=8, index_topk=16)

    def make_cache(case, offset=30000):
        return replay.make_seeded_cache(DEV, sliding_window=128, pooled_rows=case.pooled_rows, offset=offset)

    gates = (dak._ENABLED, isk._ENABLED)
    rep = replay.run_ratio4_attention_replay(attn, cache_cls=replay.SyntheticCache, make_cache=make_cache, hidden_size=256,
                                             device=DEV, repeats=3, warmup=1, pooled_rows=[96, 12], index_topk=16,
                                             stage_profile=True)
    assert (dak._ENABLED, isk._ENABLED) == gates  # the gates are put back
    assert rep["metric"] == "ds4_attention_one_layer_replay" and rep["input_tokens"] == 1
    big, small = rep["cases"]
    assert big["name"] == "ratio4_rows96_topk16" and big["median_seconds"] > 0 and big["min_seconds"] <= big["median_seconds"]
    assert rep["fused_decode_calls"] == 4  # warm-up + repeats of the one engaged case
    assert set(big["stages"]) >= {"decode_prep", "decode_sdpa", "partial_rope"}
    assert big["stages"]["decode_prep"]["calls_per_layer_call"] == 1.0
    assert big["stages"]["decode_sdpa"]["seconds_per_layer_call"] > 0
    assert "skipped" in small  # a pool not larger than the selection belongs to the composed path
    # the stage patch is gone: the module attributes are the plain functions again
    assert dak.fused_decode_prep.__name__ == "fused_decode_prep"

    rep = replay.run_ratio4_attention_replay(attn, cache_cls=replay.SyntheticCache,
                                             make_cache=lambda case: make_cache(case, offset=0), hidden_size=256,
                                             device=DEV, repeats=2, warmup=1, pooled_rows=[40], index_topk=16,
                                             stage_profile=True, input_tokens=24)
    (case,) = rep["cases"]
    assert rep["prefill_fast_calls"] == 3 and case["median_seconds"] > 0
    assert set(case["stages"]) >= {"prefill_attention", "prefill_scores", "prefill_q_qat", "topk", "partial_rope"}
    assert case["stages"]["partial_rope"]["calls_per_layer_call"] == 4.0  # q, kv, indexer q, inverse on the output
