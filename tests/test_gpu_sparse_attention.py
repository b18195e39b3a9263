"""GPU parity: indexed mixed attention decode, fused decode SDPA, batched sparse MLA decode and
the FP8-key indexer scores, against the CPU oracle on the same seeded inputs.

Tolerances are the reference's own (2e-3 max-abs for half-precision attention, 1e-5 for the
score row); recipes cite the reference test they follow.
"""

import numpy as np
import pytest
import torch

from oracle import ds4
from moespresso_amd.runtime.deepseek_v4 import decode_attention_kernel as dak
from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak
from moespresso_amd.runtime.deepseek_v4 import indexer_score_kernel as isk

pytestmark = pytest.mark.gpu


def dev():
    return torch.device("cuda:0")


def to_dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(dev())
    return t if dtype is None else t.to(dtype)


def test_indexed_decode_matches_reference_probe_shape():
    # reference tests/test_deepseek_v4_indexed_attention_kernel.py:61-89
    rng = np.random.default_rng(123)
    q = rng.standard_normal((8, 512), dtype=np.float32)
    raw = rng.standard_normal((9, 512), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((32, 512), dtype=np.float32).astype(np.float16)
    topk = np.arange(16, dtype=np.int32)
    sinks = rng.standard_normal(8, dtype=np.float32)
    got = iak.indexed_mixed_attention_decode(to_dev(q), to_dev(raw), to_dev(comp), to_dev(topk), to_dev(sinks),
                                             pos0=136).cpu().numpy()
    want = ds4.indexed_mixed_attention_decode(q, raw, comp, topk, sinks, pos0=136)
    ref = ds4.selected_rows_attention_reference(q, raw, comp, topk, sinks)
    assert got.shape == (8, 512) and got.dtype == np.float32
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3)
    np.testing.assert_allclose(got, ref, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("comp_rows", [961, 7618])
def test_indexed_decode_probe_cli_cases(comp_rows):
    # reference indexed_attention_kernel.py:2198-2216 (probe inputs): 64 heads, 128 raw rows, top-512
    rng = np.random.default_rng(comp_rows)
    q = rng.standard_normal((64, 512), dtype=np.float32)
    raw = rng.standard_normal((128, 512), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((comp_rows, 512), dtype=np.float32).astype(np.float16)
    topk = np.arange(512, dtype=np.int32)
    sinks = rng.standard_normal(64, dtype=np.float32)
    pos0 = comp_rows * 4 + 127
    got = iak.indexed_mixed_attention_decode(to_dev(q), to_dev(raw), to_dev(comp), to_dev(topk), to_dev(sinks),
                                             pos0=pos0).cpu().numpy()
    want = ds4.indexed_mixed_attention_decode(q, raw, comp, topk, sinks, pos0=pos0)
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3)


def test_indexed_decode_visit_rules():
    # negative ids skipped, first id >= visible stops the walk (reference :423-459), circular
    # raw_start (:462-503), window shorter than the ring, ratio 0, int64 topk cast, no pool rows
    rng = np.random.default_rng(5)
    q = (rng.standard_normal((16, 512)) * 0.3).astype(np.float32)
    raw = (rng.standard_normal((40, 512)) * 0.5).astype(np.float16)
    comp = (rng.standard_normal((100, 512)) * 0.5).astype(np.float16)
    sinks = rng.standard_normal(16).astype(np.float32)
    cases = [
        dict(topk=np.array([3, -1, 2, 9, 1, 0], np.int32), pos0=59, window=128, ratio=4, raw_start=0),
        dict(topk=np.array([7, 5, 99, 1], np.int32), pos0=400, window=16, ratio=4, raw_start=13),
        dict(topk=np.array([99, 0, 50], np.int32), pos0=39, window=128, ratio=0, raw_start=39),
        dict(topk=np.array([-1, -1], np.int32), pos0=80, window=8, ratio=4, raw_start=3),
        dict(topk=np.zeros((0,), np.int32), pos0=45, window=128, ratio=4, raw_start=0),
        dict(topk=np.array([50, 1], np.int32), pos0=45, window=128, ratio=4, raw_start=0),   # stops at once
    ]
    for c in cases:
        got = iak.indexed_mixed_attention_decode(to_dev(q), to_dev(raw), to_dev(comp), to_dev(c["topk"]).long(),
                                                 to_dev(sinks), pos0=c["pos0"], window=c["window"], ratio=c["ratio"],
                                                 raw_start=c["raw_start"]).cpu().numpy()
        want = ds4.indexed_mixed_attention_decode(q, raw, comp, c["topk"], sinks, pos0=c["pos0"], window=c["window"],
                                                  ratio=c["ratio"], raw_start=c["raw_start"])
        np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3, err_msg=str(c))


def test_indexed_decode_empty_softmax_gives_zeros():
    q = torch.randn((8, 512), device=dev())
    raw = torch.randn((4, 512), device=dev()).half()
    comp = torch.randn((4, 512), device=dev()).half()
    topk = torch.tensor([-1], dtype=torch.int32, device=dev())
    sinks = torch.full((8,), float("-inf"), device=dev())
    # ring deeper than pos0+1: the unsigned position arithmetic visits no raw row
    out = iak.indexed_mixed_attention_decode(q, raw, comp, topk, sinks, pos0=1)
    assert torch.all(out == 0)


def test_fused_decode_sdpa_matches_composed_chain():
    # reference tests/test_deepseek_v4_decode_attention_kernel.py:285-338
    rng = np.random.default_rng(21)
    q = (0.1 * rng.standard_normal((64, 512))).astype(np.float16)
    window = (0.1 * rng.standard_normal((128, 512))).astype(np.float16)
    row = (0.1 * rng.standard_normal(512)).astype(np.float16)
    pooled = (0.1 * rng.standard_normal((961, 512))).astype(np.float16)
    sel = np.sort(rng.choice(961, 512, replace=False)).astype(np.int32)
    sinks = rng.standard_normal(64).astype(np.float16)
    inv = ds4.rope_inverse_frequencies(64, ds4.DS4_COMPRESS_ROPE_BASE, ds4.DS4_YARN).astype(np.float32)
    params = np.array([3844, 37], dtype=np.int32)
    got = dak.fused_decode_sdpa(to_dev(q), to_dev(window), to_dev(row), to_dev(pooled), to_dev(sel), to_dev(sinks),
                                to_dev(inv), to_dev(params), scale=512 ** -0.5)
    assert got.dtype == torch.float16 and got.shape == (64, 512)
    want = ds4.fused_decode_sdpa(q, window, row, pooled, sel, sinks, inv, params, scale=512 ** -0.5)
    err = np.abs(got.float().cpu().numpy() - want.astype(np.float32)).max()
    assert err < 2e-3, err
    # the substituted row matters: a different write slot changes the result
    other = dak.fused_decode_sdpa(to_dev(q), to_dev(window), to_dev(row * 8), to_dev(pooled), to_dev(sel),
                                  to_dev(sinks), to_dev(inv), to_dev(params), scale=512 ** -0.5)
    assert not torch.equal(other, got)


@pytest.mark.parametrize("cfg", [
    dict(B=2, H=64, DK=576, dtype="bf16", n_pool=4096, n_rows=300, win=128),
    dict(B=1, H=64, DK=576, dtype="bf16", n_pool=131072, n_rows=2048, win=128),
    dict(B=3, H=128, DK=576, dtype="bf16", n_pool=2000, n_rows=77, win=0),
    dict(B=2, H=16, DK=512, dtype="f16", n_pool=999, n_rows=200, win=32),
    dict(B=1, H=7, DK=512, dtype="bf16", n_pool=64, n_rows=5, win=3),
])
def test_sparse_mla_decode_matches_oracle(cfg):
    rng = np.random.default_rng(cfg["n_rows"] + cfg["H"])
    tdt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float16
    B, H, DK, N, R, W = cfg["B"], cfg["H"], cfg["DK"], cfg["n_pool"], cfg["n_rows"], cfg["win"]
    q = to_dev(rng.standard_normal((B, H, DK), dtype=np.float32), tdt)
    kv = torch.randn((B, N, DK), device=dev(), generator=torch.Generator(device=dev()).manual_seed(7)).to(tdt)
    rows = np.stack([rng.choice(N - W, R, replace=False) for _ in range(B)]).astype(np.int32)
    rows[0, R // 2] = -1
    scale = DK ** -0.5
    got = iak.sparse_mla_decode(q, kv, to_dev(rows), scale=scale, window_start=N - W, window_rows=W)
    assert got.shape == (B, H, 512) and got.dtype == tdt
    all_rows = np.concatenate([np.tile(np.arange(N - W, N, dtype=np.int32), (B, 1)), rows], axis=1)
    gathered = np.stack([kv[b][torch.from_numpy(np.maximum(all_rows[b], 0)).to(dev()).long()].float().cpu().numpy()
                         for b in range(B)])
    # oracle on the gathered rows (ids remapped to 0..R+W-1, skipped ids stay negative)
    local = np.where(all_rows >= 0, np.arange(all_rows.shape[1])[None, :], -1)
    want = ds4.sparse_mla_decode(q.float().cpu().numpy(), gathered, local, scale=scale)
    # 2e-3 absolute plus the half-precision rounding of the output itself (short row lists give
    # outputs of magnitude ~1, where one bf16 ulp is 4e-3)
    ulp = 2.0 ** -8 if cfg["dtype"] == "bf16" else 2.0 ** -11
    err = np.abs(got.float().cpu().numpy() - want)
    assert np.all(err <= 2e-3 + ulp * np.abs(want)), err.max()


def test_sparse_mla_decode_full_config_batch16_with_sinks():
    # BASELINE config 5: 64 heads, 576/512, bf16, 131072-token cache, 2048 gathered + 128 window
    B, H, DK, N, R, W = 16, 64, 576, 131072, 2048, 128
    gen = torch.Generator(device=dev()).manual_seed(0)
    kv = torch.randn((B, N, DK), device=dev(), generator=gen, dtype=torch.float32).to(torch.bfloat16)
    q = torch.randn((B, H, DK), device=dev(), generator=gen).to(torch.bfloat16)
    rng = np.random.default_rng(0)
    ids = np.stack([np.sort(rng.choice(32768 - 32, R, replace=False)) for _ in range(B)]).astype(np.int32)
    rows = 4 * ids + 3          # compressed-entry ids address the last token of their block
    sinks = rng.standard_normal(H).astype(np.float32)
    got = iak.sparse_mla_decode(q, kv, to_dev(ids), scale=DK ** -0.5, window_start=N - W, window_rows=W,
                                sinks=to_dev(sinks), row_mul=4, row_add=3)
    all_rows = np.concatenate([np.tile(np.arange(N - W, N, dtype=np.int32), (B, 1)), rows], axis=1)
    gathered = np.stack([kv[b][torch.from_numpy(all_rows[b]).to(dev()).long()].float().cpu().numpy() for b in range(B)])
    local = np.tile(np.arange(all_rows.shape[1]), (B, 1))
    want = ds4.sparse_mla_decode(q.float().cpu().numpy(), gathered, local, scale=DK ** -0.5, sinks=sinks)
    err = np.abs(got.float().cpu().numpy() - want).max()
    assert err < 2e-3, err


def _mla_case(B, H, DK, N, R, W, seed, sinks=False, big_v=False):
    gen = torch.Generator(device=dev()).manual_seed(seed)
    kv = torch.randn((B, N, DK), device=dev(), generator=gen, dtype=torch.float32)
    if big_v:
        # columns 64..511 within +-6e4: every convex combination of them fits float16; columns 0..63 at 7e4 and
        # beyond: every convex combination of them exceeds the float16 range
        kv[..., 64:512] = (torch.rand((B, N, 448), device=dev(), generator=gen) * 2.0 - 1.0) * 6.0e4
        kv[..., :64] = kv[..., :64].abs() * 3.0e4 + 7.0e4
    kv = kv.to(torch.bfloat16)
    q = torch.randn((B, H, DK), device=dev(), generator=gen).to(torch.bfloat16)
    if big_v:
        q = (q.float() * 1.0e-4).to(torch.bfloat16)   # keeps the logits of the huge rows moderate
    rng = np.random.default_rng(seed)
    ids = np.stack([np.sort(rng.choice((N - W) // 4, R, replace=False)) for _ in range(B)]).astype(np.int32)
    snk = rng.standard_normal(H).astype(np.float32) if sinks else None
    return q, kv, ids, snk


def _mla_oracle(q, kv, ids, snk, W):
    B, N, DK = kv.shape
    rows = 4 * ids + 3
    all_rows = np.concatenate([np.tile(np.arange(N - W, N, dtype=np.int32), (B, 1)), rows], axis=1)
    gathered = np.stack([kv[b][torch.from_numpy(all_rows[b]).to(dev()).long()].float().cpu().numpy() for b in range(B)])
    local = np.tile(np.arange(all_rows.shape[1]), (B, 1))
    return ds4.sparse_mla_decode(q.float().cpu().numpy(), gathered, local, scale=DK ** -0.5, sinks=snk)


def test_sparse_mla_decode_full_config_batch4():
    # BASELINE config 5, batch 4 leg at full size (32 key ranges per sequence)
    q, kv, ids, snk = _mla_case(4, 64, 576, 131072, 2048, 128, seed=4)
    got = iak.sparse_mla_decode(q, kv, to_dev(ids), scale=576 ** -0.5, window_start=131072 - 128, window_rows=128,
                                row_mul=4, row_add=3)
    want = _mla_oracle(q, kv, ids, snk, 128)
    err = np.abs(got.float().cpu().numpy() - want).max()
    assert err < 2e-3, err


def test_sparse_mla_decode_workspace_serves_calls_of_other_shapes():
    # one workspace, sized for the largest call, reused by smaller ones (other range counts)
    from moespresso_amd import _lib
    q, kv, ids, snk = _mla_case(16, 64, 576, 8192, 500, 128, seed=11, sinks=True)
    ws = _lib.sparse_attention_workspace(16, 64, 2048 + 128, dev())
    kw = dict(scale=576 ** -0.5, window_start=8192 - 128, window_rows=128, sinks=to_dev(snk), row_mul=4, row_add=3)
    base = iak.sparse_mla_decode(q, kv, to_dev(ids), workspace=ws, **kw)
    assert np.abs(base.float().cpu().numpy() - _mla_oracle(q, kv, ids, snk, 128)).max() < 2e-3
    sub = iak.sparse_mla_decode(q[:3], kv[:3], to_dev(ids[:3, :77]), workspace=ws, **kw)
    assert np.abs(sub.float().cpu().numpy() - _mla_oracle(q[:3], kv[:3], ids[:3, :77], snk, 128)).max() < 4e-3
    assert torch.equal(iak.sparse_mla_decode(q, kv, to_dev(ids), workspace=ws, **kw), base)


def test_sparse_mla_decode_bf16_values_beyond_float16_range():
    # Per-range partial rows are stored as float16 and saturate at +-65504 (a row list served by one key
    # range is stored directly and not clamped). This pins the documented limit: columns whose V values
    # all fit float16 stay within tolerance next to columns that do not, and those come out clamped at
    # the float16 range rather than as inf/NaN.
    q, kv, ids, snk = _mla_case(2, 64, 576, 4096, 300, 128, seed=3, big_v=True)
    got = iak.sparse_mla_decode(q, kv, to_dev(ids), scale=576 ** -0.5, window_start=4096 - 128, window_rows=128,
                                row_mul=4, row_add=3).float().cpu().numpy()
    want = _mla_oracle(q, kv, ids, snk, 128)
    assert np.isfinite(got).all()
    # bf16 rounding of the output plus float16 rounding of partial rows with values up to 6e4
    bound = 2.0 ** -7 * np.abs(want) + 2.0 ** -10 * 6.0e4
    assert (np.abs(got - want)[..., 64:] <= bound[..., 64:]).all(), (np.abs(got - want) - bound)[..., 64:].max()
    assert (want[..., :64] >= 7.0e4).all()
    assert (got[..., :64] == 65536.0).all()      # 65504 rounded to bfloat16


# (the last three take the two-tiles-per-unit form of the kernel: an odd tile count, a ragged last tile,
# a ragged first half of the last unit)
@pytest.mark.parametrize("cfg", [dict(B=1, H=64, N=1000), dict(B=3, H=64, N=4099), dict(B=2, H=20, N=64),
                                 dict(B=16, H=64, N=32768), dict(B=16, H=64, N=16416), dict(B=20, H=33, N=13123),
                                 dict(B=32, H=64, N=8209), dict(B=1, H=64, N=32768)])
def test_indexer_scores_fp8_and_topk(cfg):
    B, H, N = cfg["B"], cfg["H"], cfg["N"]
    rng = np.random.default_rng(B * 1000 + N)
    q = to_dev(rng.standard_normal((B, H, 128), dtype=np.float32), torch.bfloat16)
    k32 = rng.standard_normal((B, N, 128), dtype=np.float32)
    kscale = (np.abs(k32).max(-1) / 448.0).astype(np.float32)
    codes = ds4.e4m3_encode(k32 / kscale[..., None])
    w = rng.uniform(0, 1, (B, H)).astype(np.float32)
    got = isk.indexer_scores_fp8(q, to_dev(codes).view(torch.float8_e4m3fn), to_dev(kscale), to_dev(w))
    assert got.shape == (B, N) and got.dtype == torch.float32
    want = ds4.indexer_scores_fp8(q.float().cpu().numpy(), codes, kscale, w)
    g = got.cpu().numpy()
    np.testing.assert_allclose(g, want, rtol=1e-5, atol=1e-4)
    k = min(2048, N)
    sel = isk.topk_select(got, k).cpu().numpy()
    for b in range(B):
        # indices are bit-exact for the selection rule applied to the device's own scores
        np.testing.assert_array_equal(sel[b], ds4.radix_select_topk(g[b], k))
        srt = np.sort(want[b])[::-1]
        if k < N and srt[k - 1] - srt[k] > 1e-3:
            assert set(sel[b].tolist()) == set(ds4.radix_select_topk(want[b].astype(np.float32), k).tolist())


def test_indexer_scores_fp8_exact_integer_case():
    # integer queries and small-integer keys: every sum is exact in float32, so device scores equal
    # the float64 closed form bit for bit and top-k indices (many ties) match the oracle end to end
    rng = np.random.default_rng(4)
    B, H, N = 2, 64, 5000
    qi = rng.integers(-2, 3, (B, H, 128)).astype(np.float32)
    ki = rng.integers(-3, 4, (B, N, 128)).astype(np.float32)
    codes = ds4.e4m3_encode(ki)
    kscale = np.full((B, N), 0.5, dtype=np.float32)
    w = (rng.integers(0, 5, (B, H)) * 0.25).astype(np.float32)
    got = isk.indexer_scores_fp8(to_dev(qi, torch.bfloat16), to_dev(codes), to_dev(kscale), to_dev(w))
    want = ds4.indexer_scores_fp8(qi, codes, kscale, w).astype(np.float32)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    sel = isk.topk_select(got, 2048).cpu().numpy()
    for b in range(B):
        np.testing.assert_array_equal(sel[b], ds4.radix_select_topk(want[b], 2048))
