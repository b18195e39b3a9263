"""GPU parity: prefill-side DS4 consumers (through the C-ABI) vs the NumPy oracle.

Shapes follow the reference's tests/test_deepseek_v4_indexed_attention_kernel.py (:92-310, :372-505,
:571-765); tolerance for the attention forms is the reference's own 2e-3 (rtol = atol).
"""

import numpy as np
import pytest
import torch

from oracle import ds4

pytestmark = pytest.mark.gpu


def _dev():
    return torch.device("cuda:0")


def _t(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(_dev())


def _live_case(tokens, n_comp, heads=64, seed=99, raw_cap=None, width=None, batch=1):
    """The reference's _live_prefill_case recipe (:289-308), optionally with a deeper ring."""
    rng = np.random.default_rng(seed)
    raw_cap = tokens if raw_cap is None else raw_cap
    q = rng.standard_normal((batch, heads, tokens, 512), dtype=np.float32)
    raw = rng.standard_normal((batch, 1, raw_cap, 512), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((batch, n_comp, 512), dtype=np.float32).astype(np.float16)
    width = min(512, n_comp) if width is None else width
    ids = np.stack([[np.sort(rng.choice(n_comp, size=width, replace=False)) for _ in range(tokens)]
                    for _ in range(batch)]).astype(np.int32)
    sinks = rng.standard_normal((heads,), dtype=np.float32)
    return q, raw, comp, ids, sinks


def _oracle_live(q, raw, comp, ids, sinks, **kw):
    out = np.empty(q.shape, dtype=np.float64)
    for b in range(q.shape[0]):
        o = ds4.indexed_mixed_attention_prefill(q[b].transpose(1, 0, 2), raw[b, 0], comp[b], ids[b], sinks, **kw)
        out[b] = o.transpose(1, 0, 2)
    return out


def test_prefill_probe_layout_matches_oracle():
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    rng = np.random.default_rng(456)  # reference :97-105
    q = rng.standard_normal((3, 8, 512), dtype=np.float32)
    raw = rng.standard_normal((3, 512), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((12, 512), dtype=np.float32).astype(np.float16)
    topk = np.tile(np.arange(8, dtype=np.int32), (3, 1))
    sinks = rng.standard_normal((8,), dtype=np.float32)
    got = iak.indexed_mixed_attention_prefill(_t(q), _t(raw), _t(comp), _t(topk), _t(sinks), pos0=0, window=128)
    want = ds4.indexed_mixed_attention_prefill(q, raw, comp, topk, sinks, pos0=0, window=128)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("tokens,n_comp", [(200, 50), (137, 34), (96, 512)])
@pytest.mark.parametrize("q_dtype", [torch.float32, torch.float16])
def test_prefill_live_matches_oracle(tokens, n_comp, q_dtype):
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    q, raw, comp, ids, sinks = _live_case(tokens, n_comp)
    fn = iak.indexed_mixed_attention_prefill_live_f32 if q_dtype == torch.float32 else \
        iak.indexed_mixed_attention_prefill_live_f16
    qt = _t(q, q_dtype)
    got = fn(qt, _t(raw), _t(comp), _t(ids), _t(sinks), pos0=0, window=128, ratio=4)
    assert got.dtype == torch.float32 and tuple(got.shape) == q.shape
    want = _oracle_live(qt.float().cpu().numpy(), raw, comp, ids, sinks, pos0=0, window=128, ratio=4)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=2e-3, atol=2e-3)


def _oracle_tokens(q, raw, comp, ids, sinks, tokens, *, pos0, window, ratio, raw_start=0):
    """Oracle rows of the sampled tokens of batch entry 0 (q is BHLD): the per-token visit rules with the
    chunk's newest ring row at pos0 + T - 1, then float64 sink attention on float16-rounded queries."""
    T = q.shape[2]
    out = {}
    for t in tokens:
        raw_rows, comp_rows = ds4.indexed_visit_rows(
            raw_cap=raw.shape[2], n_comp=comp.shape[1], topk=ids[0, t], qpos=pos0 + t, last_pos=pos0 + T - 1,
            window=window, ratio=ratio, raw_start=raw_start)
        rows = np.concatenate([raw[0, 0, raw_rows].astype(np.float32).reshape(-1, 512),
                               comp[0, comp_rows].astype(np.float32).reshape(-1, 512)], axis=0)
        out[t] = ds4.attend_rows_f64(ds4.round_f16(q[0, :, t].astype(np.float32)), rows, sinks, 512 ** -0.5)
    return out


@pytest.mark.parametrize("q_dtype", [torch.float16, torch.float32])
def test_prefill_live_at_the_anchor_chunk(q_dtype):
    """The reference's anchor chunk: 3844 tokens, 64 heads, top-512 of the pool, window 128, here from
    position 5000 on a ring deeper than the chunk with a rotated start, and a pool that becomes visible
    while the chunk proceeds (ids ascending; the walk stops at the first invisible one). Sampled tokens
    against the oracle; both query types run on the persistent consumer."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    T, P, pos0, raw_cap, raw_start = 3844, 2300, 5000, 3900, 1234
    rng = np.random.default_rng(2024)
    q = rng.standard_normal((1, 64, T, 512), dtype=np.float32)
    if q_dtype == torch.float16:
        q = q.astype(np.float16)
    raw = rng.standard_normal((1, 1, raw_cap, 512), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((1, P, 512), dtype=np.float32).astype(np.float16)
    ids = np.stack([np.sort(rng.choice(P, size=512, replace=False)) for _ in range(T)])[None].astype(np.int32)
    sinks = rng.standard_normal((64,), dtype=np.float32)
    kw = dict(pos0=pos0, window=128, ratio=4, raw_start=raw_start)
    fn = iak.indexed_mixed_attention_prefill_live_f16 if q_dtype == torch.float16 else \
        iak.indexed_mixed_attention_prefill_live_f32
    got = fn(_t(q), _t(raw), _t(comp), _t(ids), _t(sinks), **kw).cpu().numpy()
    tokens = [0, 1, 63, 127, 128, 129, 1000, 1921, 2500, 3000, 3842, 3843]
    want = _oracle_tokens(q, raw, comp, ids, sinks, tokens, **kw)
    for t in tokens:
        np.testing.assert_allclose(got[0, :, t], want[t], rtol=2e-3, atol=2e-3, err_msg=f"token {t}")
    assert np.isfinite(got).all()


@pytest.mark.parametrize("q_dtype", [torch.float16, torch.float32])
def test_banded_prefill_at_the_anchor_chunk(q_dtype):
    """The banded route at the anchor chunk: 3844 tokens from position 5000, a band of 128 positions and every
    pool row visible at ratio 128 (ascending ids over the whole pool, of which a token sees the first
    (position + 1) / 128). Sampled tokens against the oracle."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    T, pos0, ratio = 3844, 5000, 128
    P = (pos0 + T) // ratio
    rng = np.random.default_rng(2025)
    q = rng.standard_normal((1, 64, T, 512), dtype=np.float32)
    if q_dtype == torch.float16:
        q = q.astype(np.float16)
    raw = rng.standard_normal((1, 1, T, 512), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((1, P, 512), dtype=np.float32).astype(np.float16)
    ids = np.ascontiguousarray(np.broadcast_to(np.arange(P, dtype=np.int32), (1, T, P)))
    sinks = rng.standard_normal((64,), dtype=np.float32)
    kw = dict(pos0=pos0, window=128, ratio=ratio)
    got = iak.banded_prefill_attention_live(_t(q), _t(raw), _t(comp), _t(ids), _t(sinks), **kw).cpu().numpy()
    tokens = [0, 1, 119, 120, 127, 128, 1000, 2000, 3715, 3716, 3842, 3843]
    want = _oracle_tokens(q, raw, comp, ids, sinks, tokens, **kw)
    for t in tokens:
        np.testing.assert_allclose(got[0, :, t], want[t], rtol=2e-3, atol=2e-3, err_msg=f"token {t}")
    assert np.isfinite(got).all()


def test_prefill_live_more_than_1024_keys_per_token():
    """window + top_k beyond one workgroup's slot table: every token is split into key ranges and merged
    with token strides."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    T, P, pos0 = 300, 1500, 7000
    rng = np.random.default_rng(7)
    q = rng.standard_normal((1, 32, T, 512), dtype=np.float32)
    raw = rng.standard_normal((1, 1, 900, 512), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((1, P, 512), dtype=np.float32).astype(np.float16)
    ids = np.stack([np.sort(rng.choice(P, size=512, replace=False)) for _ in range(T)])[None].astype(np.int32)
    sinks = rng.standard_normal((32,), dtype=np.float32)
    kw = dict(pos0=pos0, window=600, ratio=4, raw_start=77)
    got = iak.indexed_mixed_attention_prefill_live_f32(_t(q), _t(raw), _t(comp), _t(ids), _t(sinks), **kw).cpu().numpy()
    tokens = [0, 1, 150, 298, 299]
    want = _oracle_tokens(q, raw, comp, ids, sinks, tokens, **kw)
    for t in tokens:
        np.testing.assert_allclose(got[0, :, t], want[t], rtol=2e-3, atol=2e-3, err_msg=f"token {t}")


def test_composed_reference_forms_agree_with_the_kernels():
    """The two composed reference forms the reference module carries (:2111, :2133) against the kernels, as
    its own tests use them (tolerance 2e-3)."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    rng = np.random.default_rng(31)
    q = rng.standard_normal((24, 16, 512), dtype=np.float32)
    raw = rng.standard_normal((24, 512), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((40, 512), dtype=np.float32).astype(np.float16)
    ids = np.stack([np.sort(rng.choice(40, size=12, replace=False)) for _ in range(24)]).astype(np.int32)
    sinks = rng.standard_normal((16,), dtype=np.float32)
    args = (_t(q), _t(raw), _t(comp), _t(ids), _t(sinks))
    ref = iak.mlx_indexed_mixed_attention_prefill_reference(*args, pos0=60, window=8, ratio=4)
    got = iak.indexed_mixed_attention_prefill(*args, pos0=60, window=8, ratio=4)
    np.testing.assert_allclose(got.cpu().numpy(), ref.cpu().numpy(), rtol=2e-3, atol=2e-3)
    np.testing.assert_allclose(ref.cpu().numpy(), ds4.indexed_mixed_attention_prefill_reference(
        q, raw, comp, ids, sinks, pos0=60, window=8, ratio=4), rtol=1e-4, atol=1e-5)
    one = iak.mlx_selected_rows_attention_reference(_t(q[0]), _t(raw), _t(comp), _t(ids[0]), _t(sinks))
    dec = iak.indexed_mixed_attention_decode(_t(q[0]), _t(raw), _t(comp), _t(ids[0]), _t(sinks), pos0=40 * 4 + 23,
                                             window=128)
    np.testing.assert_allclose(dec.cpu().numpy(), one.cpu().numpy(), rtol=2e-3, atol=2e-3)


def test_prefill_live_negative_and_stop_ids_offset_chunk_and_ring():
    """Negative ids are skipped, the first invisible id ends the walk, the chunk starts at pos0 > 0 and the
    ring is deeper than the chunk with a rotated start (reference :423-505)."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    tokens, n_comp, raw_cap = 40, 64, 72
    q, raw, comp, ids, sinks = _live_case(tokens, n_comp, heads=16, seed=5, raw_cap=raw_cap, width=24, batch=2)
    rng = np.random.default_rng(6)
    ids = rng.integers(0, n_comp, size=ids.shape).astype(np.int32)  # unsorted: break rule matters
    ids[:, ::3, 2] = -1
    ids[:, ::5, 7] = -7
    kw = dict(pos0=100, window=16, ratio=4, raw_start=50)
    got = iak.indexed_mixed_attention_prefill_live_f32(_t(q), _t(raw), _t(comp), _t(ids), _t(sinks), **kw)
    want = _oracle_live(q, raw, comp, ids, sinks, **kw)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=2e-3, atol=2e-3)


def test_banded_prefill_matches_oracle_and_zero_pool():
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    tokens, n_comp = 150, 9
    q, raw, comp, _, sinks = _live_case(tokens, n_comp, heads=32, seed=8)
    ids = np.tile(np.arange(n_comp, dtype=np.int32), (1, tokens, 1))  # ascending: attend every visible pool row
    kw = dict(pos0=0, window=64, ratio=16)
    got = iak.banded_prefill_attention_live(_t(q), _t(raw), _t(comp), _t(ids), _t(sinks), **kw)
    want = _oracle_live(q, raw, comp, ids, sinks, **kw)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=2e-3, atol=2e-3)
    # zero-pool layer: one dummy pool row, zero-width topk (reference :612-683)
    empty = np.zeros((1, tokens, 0), dtype=np.int32)
    got0 = iak.banded_prefill_attention_live(_t(q), _t(raw), _t(comp[:, :1]), _t(empty), _t(sinks), **kw)
    want0 = _oracle_live(q, raw, comp[:, :1], empty, sinks, **kw)
    np.testing.assert_allclose(got0.cpu().numpy(), want0, rtol=2e-3, atol=2e-3)


def test_prefill_consumer_counters_and_rejections(monkeypatch):
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    q, raw, comp, ids, sinks = _live_case(8, 8, heads=16, seed=1)
    args = (_t(q), _t(raw), _t(comp), _t(ids), _t(sinks))
    before = iak.prefill_consumer_call_counts()
    iak.indexed_mixed_attention_prefill_live_f32(*args, pos0=0)
    monkeypatch.setenv("MOESPRESSO_DSV4_R4_PREFILL_CONSUMER_MMA", "0")
    iak.indexed_mixed_attention_prefill_live_f32(*args, pos0=0)  # 16 heads, no mma, not % 32 -> v1
    after = iak.prefill_consumer_call_counts()
    assert after["mma"] == before["mma"] + 1 and after["v1"] == before["v1"] + 1
    with pytest.raises(ValueError, match="mma consumer"):
        iak.banded_prefill_attention_live(*args, pos0=0, window=8, ratio=4)
    monkeypatch.delenv("MOESPRESSO_DSV4_R4_PREFILL_CONSUMER_MMA")
    with pytest.raises(ValueError, match="positive window and ratio"):
        iak.banded_prefill_attention_live(*args, pos0=0, window=0, ratio=4)
    with pytest.raises(ValueError, match="divisible by 8"):
        iak.indexed_mixed_attention_prefill_live_f32(_t(q[:, :12]), *args[1:4], _t(sinks[:12]), pos0=0)
    with pytest.raises(ValueError, match="float16 or float32"):
        iak.banded_prefill_attention_live(_t(q, torch.bfloat16), *args[1:], pos0=0, window=8, ratio=4)
    with pytest.raises(ValueError, match="at least one row"):
        iak.banded_prefill_attention_live(args[0], args[1], _t(comp[:, :0]), args[3], args[4], pos0=0, window=8,
                                          ratio=4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_indexer_scores_tiled_live(dtype):
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    rng = np.random.default_rng(321)  # reference :240-247, plus a second batch entry and a larger pool
    # (the last two: several tiles per workgroup with the visible prefix ending inside a block; five tiles per
    # workgroup, all visible, a ragged last block)
    for (B, H, T, P, pos0) in ((1, 8, 5, 19, 0), (2, 64, 37, 300, 250), (1, 48, 9, 33, 1000), (1, 64, 130, 1000, 1500),
                               (1, 64, 300, 1500, 9000)):
        q = rng.standard_normal((B, H, T, 128), dtype=np.float32)
        w = (rng.standard_normal((B, T, H), dtype=np.float32) * (H ** -0.5) * (128 ** -0.5)).astype(np.float32)
        comp = rng.standard_normal((B, P, 128), dtype=np.float32)
        qt, ct = _t(q, dtype), _t(comp, dtype)
        before = iak.indexer_scores_call_counts()
        got = iak.indexer_scores_tiled_live(qt, _t(w), ct, pos0=pos0, ratio=4).cpu().numpy()
        after = iak.indexer_scores_call_counts()
        key = "f16" if dtype == torch.float16 else "f32"
        assert after[key] == before[key] + 1
        want = ds4.indexer_scores_tiled_live(qt.float().cpu().numpy(), w, ct.float().cpu().numpy(), pos0=pos0, ratio=4)
        inf = np.isinf(want)
        assert (np.isinf(got) == inf).all() and (got[inf] < 0).all()
        np.testing.assert_allclose(got[~inf], want[~inf], rtol=1e-4, atol=1e-4)
    with pytest.raises(ValueError, match="both q and index_comp as float16"):
        iak.indexer_scores_tiled_live(_t(q, torch.float16), _t(w), _t(comp), pos0=0)
    with pytest.raises(ValueError, match="weights must be float32"):
        iak.indexer_scores_tiled_live(_t(q), _t(w, torch.float16), _t(comp), pos0=0)


def test_indexer_scores_tiled_live_at_the_anchor_chunk():
    """3844 tokens x 961 pool rows x 64 heads, float16 operands (the served form); sampled tokens against the
    oracle, each as a one-token chunk at its own position."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    T, P, H, pos0 = 3844, 961, 64, 0
    rng = np.random.default_rng(11)
    q = rng.standard_normal((1, H, T, 128), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((1, P, 128), dtype=np.float32).astype(np.float16)
    w = (rng.standard_normal((1, T, H), dtype=np.float32) * (H ** -0.5) * (128 ** -0.5)).astype(np.float32)
    got = iak.indexer_scores_tiled_live(_t(q), _t(w), _t(comp), pos0=pos0, ratio=4).cpu().numpy()
    assert got.shape == (1, T, P)
    for t in (0, 2, 3, 4, 500, 1921, 3000, 3843):
        want = ds4.indexer_scores_tiled_live(q[:, :, t:t + 1].astype(np.float32), w[:, t:t + 1],
                                             comp.astype(np.float32), pos0=pos0 + t, ratio=4)[0, 0]
        inf = np.isinf(want)
        assert inf.sum() == P - min((pos0 + t + 1) // 4, P)
        assert (np.isinf(got[0, t]) == inf).all()
        np.testing.assert_allclose(got[0, t][~inf], want[~inf], rtol=1e-4, atol=1e-4, err_msg=f"token {t}")


def test_indexer_scores_tiled_live_f16_operands_bit_identical():
    """Float16 operands carry the values the float32 form stages, so the two forms agree bit for bit
    (reference :856-875)."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    rng = np.random.default_rng(77)
    q = rng.standard_normal((1, 64, 21, 128), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((1, 130, 128), dtype=np.float32).astype(np.float16)
    w = rng.uniform(0, 1, (1, 21, 64)).astype(np.float32)
    a = iak.indexer_scores_tiled_live(_t(q), _t(w), _t(comp), pos0=600)
    b = iak.indexer_scores_tiled_live(_t(q.astype(np.float32)), _t(w), _t(comp.astype(np.float32)), pos0=600)
    assert torch.equal(a, b)


def test_indexer_q_qat_live_bit_exact_and_matches_decode_contract():
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    rng = np.random.default_rng(654)  # reference :272-274
    q = np.ascontiguousarray(rng.standard_normal((1, 4, 8, 128), dtype=np.float32).transpose(0, 2, 1, 3))
    got = iak.indexer_q_qat_live(_t(q)).cpu().numpy()
    np.testing.assert_array_equal(got, ds4.indexer_q_qat_live(q))
    np.testing.assert_allclose(got, ds4.indexer_qat(q), rtol=1e-5, atol=1e-5)  # the reference's own check
    big = (rng.standard_normal((2, 16, 33, 128)) * np.exp(rng.uniform(-20, 20, (2, 16, 33, 1)))).astype(np.float32)
    np.testing.assert_array_equal(iak.indexer_q_qat_live(_t(big)).cpu().numpy(), ds4.indexer_q_qat_live(big))
    with pytest.raises(ValueError, match="q must be float32"):
        iak.indexer_q_qat_live(_t(q, torch.float16))
