"""Eligibility order of the fused ratio-4 decode wrapper on CPU tensors (no kernel runs): every miss
delegates to the wrapped block before any cache mutation (reference model.py:1551-1607; test
tests/test_deepseek_v4_decode_attention_kernel.py:532-578)."""

import torch

from ds4_standins import Attention, Cache, OtherCache, steady_cache
from moespresso_amd.runtime.deepseek_v4 import decode_attention_kernel as dak
from moespresso_amd.runtime.deepseek_v4 import model as dsm


def _marked(**kw):
    cache = steady_cache("cpu", **kw)
    object.__setattr__(cache, "_moespresso_dsv4_fp8_kv_cache", True)
    return cache


def test_every_contract_miss_delegates_before_touching_the_cache(monkeypatch):
    monkeypatch.setattr(dak, "fused_decode_enabled", lambda: True)
    attn = Attention("cpu")
    wrapper = dsm._Ratio4DecodeFusedAttention(attn, cache_cls=Cache)
    x = torch.zeros((1, 1, 256), dtype=torch.float16)
    good = _marked(rows=96)
    assert wrapper._decode_eligible(x, good)

    misses = []
    misses.append((torch.zeros((1, 4, 256), dtype=torch.float16), good))          # prefill shape
    misses.append((torch.zeros((2, 1, 256), dtype=torch.float16), good))          # batch
    misses.append((x.float(), good))                                              # element type
    misses.append((x, steady_cache("cpu", rows=96)))                              # cache without the rounded append
    misses.append((x, _marked(rows=96, cls=OtherCache)))                          # another cache class
    misses.append((x, _marked(rows=96, offset=100)))                              # ring not yet full
    odd_keep = _marked(rows=96)
    odd_keep.local.keep = 4
    misses.append((x, odd_keep))                                                  # ring keeps a prefix
    f32_ring = _marked(rows=96)
    f32_ring.local.keys = f32_ring.local.keys.float()
    misses.append((x, f32_ring))                                                  # ring element type
    short = _marked(rows=96)
    short.local.max_size = 64
    misses.append((x, short))                                                     # ring size != sliding window
    for xi, cache in misses:
        assert not wrapper._decode_eligible(xi, cache)
        wrapper(xi, mask=None, cache=cache)
    assert len(attn.stock_calls) == len(misses)
    assert attn.compressor.calls == [] and wrapper.fused_decode_calls == 0

    # geometry of the wrapped block
    for name, value in (("compress_ratio", 128), ("head_dim", 256)):
        other = Attention("cpu")
        setattr(other, name, value)
        assert not dsm._Ratio4DecodeFusedAttention(other, cache_cls=Cache)._decode_eligible(x, good)
    other = Attention("cpu")
    other.indexer.index_topk = 0
    assert not dsm._Ratio4DecodeFusedAttention(other, cache_cls=Cache)._decode_eligible(x, good)
    other = Attention("cpu")
    other.rope.dims = 32
    assert not dsm._Ratio4DecodeFusedAttention(other, cache_cls=Cache)._decode_eligible(x, good)

    # debug dumps veto the fused path; the gate itself too
    monkeypatch.setenv("MOESPRESSO_DSV4_INDEXER_DUMP_PREFIX", "/tmp/x")
    assert not wrapper._decode_eligible(x, good)
    monkeypatch.delenv("MOESPRESSO_DSV4_INDEXER_DUMP_PREFIX")
    monkeypatch.setattr(dak, "fused_decode_enabled", lambda: False)
    assert not wrapper._decode_eligible(x, good)


def test_score_contract_decides_before_the_compressor_moves(monkeypatch):
    # A decode token the contract does not serve (gate off, no device, geometry) must reach the wrapped
    # indexer with the compressor untouched: the wrapped indexer advances it itself, and a second advance
    # for the same token corrupts the pool (reference model.py:870-1056 never re-enters).
    from moespresso_amd.runtime.deepseek_v4 import indexer_score_kernel as isk

    attn = Attention("cpu", index_heads=64, topk=16)
    contract = dsm._IndexerDS4ScoreContract(attn.indexer, 4, layer_index=0)
    cache = steady_cache("cpu", rows=40)
    x = torch.zeros((1, 1, 256), dtype=torch.float16)
    q_res = torch.zeros((1, 1, 64), dtype=torch.float16)
    monkeypatch.setattr(isk, "_ENABLED", False)
    assert contract(x, q_res, None, None, cache, 100) is None
    monkeypatch.setattr(isk, "_ENABLED", True)
    monkeypatch.setattr(isk, "_metal_available", lambda: False)
    assert contract(x, q_res, None, None, cache, 101) is None
    monkeypatch.setattr(isk, "_metal_available", lambda: True)
    attn.indexer.head_dim = 64                                   # geometry the score kernel does not serve
    assert contract(x, q_res, None, None, cache, 102) is None
    attn.indexer.head_dim = 128
    assert contract(torch.zeros((1, 3, 256), dtype=torch.float16), q_res, None, None, cache, 103) is None
    assert attn.indexer.stock_calls == 4
    # one advance per token, all of them the wrapped indexer's own
    assert attn.indexer.compressor.positions == [100, 101, 102, 103] and cache.indexer_state["advances"] == 4
    c = "_moespresso_dsv4_indexer_score_contract_"
    assert getattr(contract, c + "calls") == 0


def test_score_tail_gates(monkeypatch):
    # reference indexer_score_kernel.py:499-560: two env kill switches read per call, then shape and type
    from moespresso_amd.runtime.deepseek_v4 import indexer_score_kernel as isk

    monkeypatch.setattr(isk, "_metal_available", lambda: True)
    assert isk.score_tail_enabled()
    for env in ("MOESPRESSO_DSV4_INDEXER_CHAIN_TRIMS", "MOESPRESSO_DSV4_INDEXER_SCORE_TAIL"):
        monkeypatch.setenv(env, "0")
        assert not isk.score_tail_enabled()
        monkeypatch.setenv(env, "1")
        assert isk.score_tail_enabled()
        monkeypatch.delenv(env)
    scores = torch.zeros((1, 64, 1, 96))
    w = torch.zeros((1, 1, 64), dtype=torch.bfloat16)
    params = torch.tensor([7, 50], dtype=torch.int32)
    assert isk.score_tail_eligible(scores, w, params)
    assert isk.score_tail_eligible(torch.zeros((1, 32, 1, 1)), torch.zeros((1, 1, 32)), params)
    assert not isk.score_tail_eligible(torch.zeros((1, 31, 1, 96)), torch.zeros((1, 1, 31)), params)   # < 32 heads
    assert not isk.score_tail_eligible(torch.zeros((1, 65, 1, 96)), torch.zeros((1, 1, 65)), params)   # > 64 heads
    assert not isk.score_tail_eligible(torch.zeros((2, 64, 1, 96)), w, params)                          # batch
    assert not isk.score_tail_eligible(torch.zeros((1, 64, 2, 96)), w, params)                          # tokens
    assert not isk.score_tail_eligible(torch.zeros((1, 64, 1, 0)), w, params)                           # empty
    assert not isk.score_tail_eligible(scores.half(), w, params)                                        # score type
    assert not isk.score_tail_eligible(scores, torch.zeros((1, 64)), params)                            # weight rank
    assert not isk.score_tail_eligible(scores, torch.zeros((1, 1, 63)), params)                         # weight shape
    assert not isk.score_tail_eligible(scores, w.double(), params)                                      # weight type
    assert not isk.score_tail_eligible(scores, w, params.long())                                        # params type
    assert not isk.score_tail_eligible(scores, w, params[:1])                                           # params size
    monkeypatch.setattr(isk, "_metal_available", lambda: False)
    assert not isk.score_tail_enabled() and not isk.score_tail_eligible(scores, w, params)


def test_row_helpers_accept_the_reference_module_handle(monkeypatch):
    # reference model.py:745,752,772 are called as f(mx, x)
    from moespresso_amd.runtime.deepseek_v4 import indexer_score_kernel as isk

    seen = []
    monkeypatch.setattr(isk, "indexer_qat_rows", lambda rows: seen.append(rows) or rows)
    x = torch.zeros((2, 128))
    assert dsm._dsv4_indexer_qat(x) is x and dsm._dsv4_indexer_qat(torch, x) is x
    assert dsm._dsv4_prefill_pooled_qat(torch, x) is x
    rows, used = dsm._dsv4_decode_indexer_qat(torch, x)
    assert rows is x and used and len(seen) == 4
    import pytest
    with pytest.raises(TypeError):
        dsm._dsv4_indexer_qat(x, x)


def test_cache_wrappers_are_idempotent_and_keep_the_originals():
    cache = steady_cache("cpu", rows=4)
    original = cache.update_and_fetch
    dsm._cache_with_fp8_kv_roundtrip(cache)
    dsm._cache_with_fp8_kv_roundtrip(cache)
    assert getattr(cache, dsm._CACHE_WRAPPER_ORIGINALS_ATTR)["update_and_fetch"] == original
    dsm._cache_with_compressed_pool_aux_trim_clear(cache)
    dsm._cache_with_compressed_pool_aux_trim_clear(cache)
    assert set(getattr(cache, dsm._CACHE_WRAPPER_ORIGINALS_ATTR)) == {"update_and_fetch", "trim"}
    # rows of another width pass through the wrapped update untouched (no kernel involved)
    rows = torch.zeros((1, 1, 2, 128))
    k, v = cache.update_and_fetch(rows, rows)
    assert k is rows and v is rows and cache.update_calls == 1


def test_replay_case_selection_and_rope_frequencies():
    import numpy as np

    from moespresso_amd.runtime.deepseek_v4 import ratio4_attention_replay as replay
    from oracle import ds4

    cases = replay.default_replay_cases()
    assert [c.pooled_rows for c in cases] == [0, 961, 7618, 961, 512] and not cases[0].cache
    assert replay.selected_replay_cases(include_splits=False) == cases[:3]
    assert replay.selected_replay_cases(include_splits=True) == cases
    picked = replay.selected_replay_cases(include_splits=False, pooled_rows=[100, 200], index_topk=64)
    assert [c.name for c in picked] == ["ratio4_rows100_topk64", "ratio4_rows200_topk64"]
    yarn = {"factor": 16.0, "original_seq_len": 65536, "beta_fast": 32, "beta_slow": 1}
    for base, y in ((10000.0, None), (160000.0, yarn)):
        np.testing.assert_array_equal(replay.rope_inverse_frequencies(64, base, y).numpy(),
                                      ds4.rope_inverse_frequencies(64, base, y).astype(np.float32))
