"""GPU parity: DS4 indexer QAT, score row, score tail, FP8 rows, prep, top-k.

Every test calls the HIP kernels through the Python operator modules (which go
through the C-ABI) and compares with the CPU oracle on the same seeded inputs.
Recipes follow the reference's tests (cited per test).
"""

import numpy as np
import pytest
import torch

from oracle import ds4
from moespresso_amd.runtime.deepseek_v4 import decode_attention_kernel as dak
from moespresso_amd.runtime.deepseek_v4 import indexer_score_kernel as isk

pytestmark = pytest.mark.gpu


def dev():
    return torch.device("cuda:0")


def to_dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(dev())
    return t if dtype is None else t.to(dtype)


def bits(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32)).view(np.uint32)


def _qat_case_rows(name, rng):
    # reference tests/test_deepseek_v4_indexer_score_kernel.py:36-71
    if name == "normal":
        return rng.standard_normal((1024, 128)).astype(np.float32)
    if name == "scaled_2p30":
        return (rng.standard_normal((1024, 128)) * 2.0 ** 30).astype(np.float32)
    if name == "scaled_2m30":
        return (rng.standard_normal((1024, 128)) * 2.0 ** -30).astype(np.float32)
    if name == "amax_near_lattice_boundary":
        base = rng.standard_normal((1024, 128)).astype(np.float32)
        groups = base.reshape(1024, 4, 32)
        amax = np.abs(groups).max(axis=-1, keepdims=True)
        target = 6.0 * (2.0 ** rng.integers(-40, 40, size=(1024, 4, 1)))
        jitter = 1.0 + rng.integers(-4, 5, size=(1024, 4, 1)) * np.float32(1.1920929e-07)
        return (groups / amax * target * jitter).astype(np.float32).reshape(1024, 128)
    if name == "lattice_midpoints":
        mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
        signs = np.where(rng.random((256, 128)) < 0.5, 1.0, -1.0)
        return (rng.choice(mids, size=(256, 128)) * signs).astype(np.float32)
    if name == "zeros_and_denormals":
        rows = np.zeros((8, 128), dtype=np.float32)
        rows[1] = -0.0
        rows[2] = 1e-39
        rows[3] = rng.standard_normal(128) * 1e-38
        rows[4] = rng.standard_normal(128) * 1e-44
        return rows
    if name == "one_hot_power_of_two":
        # post-Hadamard rows are constant +-2^k*128^-1/2: group amax sits exactly on the
        # lattice/scale boundaries for many exponents
        rows = np.zeros((160, 128), dtype=np.float32)
        for i in range(160):
            rows[i, i % 128] = 2.0 ** (i - 80)
        return rows
    raise AssertionError(name)


@pytest.mark.parametrize("case", ["normal", "scaled_2p30", "scaled_2m30", "amax_near_lattice_boundary",
                                  "lattice_midpoints", "zeros_and_denormals", "one_hot_power_of_two"])
def test_indexer_qat_rows_bitexact_float32(case):
    rows = _qat_case_rows(case, np.random.default_rng(1234))
    got = isk.indexer_qat_rows(to_dev(rows)).cpu().numpy()
    want = ds4.indexer_qat(rows)
    assert got.dtype == np.float32
    np.testing.assert_array_equal(bits(got), bits(want))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_indexer_qat_rows_bitexact_low_precision_query(dtype):
    # reference :101-123
    rng = np.random.default_rng(77)
    rows = to_dev(rng.standard_normal((1, 64, 1, 128), dtype=np.float32), dtype)
    got = isk.indexer_qat_rows(rows)
    assert got.shape == rows.shape and got.dtype == torch.float32
    want = ds4.indexer_qat(rows.float().cpu().numpy())
    np.testing.assert_array_equal(bits(got.cpu().numpy()), bits(want))


def test_indexer_qat_of_ones_known_answer():
    got = isk.indexer_qat_rows(torch.ones((3, 128), device=dev())).cpu().numpy()
    want = np.zeros((3, 128), dtype=np.float32)
    want[:, 0] = 12.0
    np.testing.assert_array_equal(got, want)


def _score_inputs(n_rows, rng, n_heads=64, q_dtype=np.float32):
    # reference :21-35
    q = rng.standard_normal((1, n_heads, 1, 128), dtype=np.float32)
    pooled = ds4.indexer_qat(rng.standard_normal((1, n_rows, 128), dtype=np.float32))
    w = (rng.standard_normal((1, 1, n_heads), dtype=np.float32) * n_heads ** -0.5).astype(np.float32)
    return q, pooled, w


@pytest.mark.parametrize("n_rows", [3, 512, 961, 977, 4099])
def test_fused_qat_indexer_scores_matches_composed_chain(n_rows):
    # reference :137-163: rtol=atol=1e-5 and identical top-512 set
    rng = np.random.default_rng(1000 + n_rows)
    q, pooled, w = _score_inputs(n_rows, rng)
    scale = 128 ** -0.5
    got = isk.fused_qat_indexer_scores(to_dev(q), to_dev(pooled), to_dev(w), scale).cpu().numpy()
    want = ds4.fused_qat_indexer_scores(q, pooled, w, scale)
    assert got.shape == (n_rows,)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    k = min(512, n_rows)
    assert set(np.argpartition(-got, k - 1)[:k].tolist()) == set(np.argpartition(-want, k - 1)[:k].tolist())


def test_fused_qat_indexer_scores_low_precision_and_few_heads():
    rng = np.random.default_rng(9)
    q, pooled, w = _score_inputs(961, rng)
    qh = to_dev(q, torch.float16)
    got = isk.fused_qat_indexer_scores(qh, to_dev(pooled), to_dev(w), 128 ** -0.5).cpu().numpy()
    want = ds4.fused_qat_indexer_scores(qh.float().cpu().numpy(), pooled, w, 128 ** -0.5)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    rng = np.random.default_rng(42)
    q, pooled, w = _score_inputs(5, rng, n_heads=1)
    got = isk.fused_qat_indexer_scores(to_dev(q), to_dev(pooled), to_dev(w), 128 ** -0.5).cpu().numpy()
    np.testing.assert_allclose(got, ds4.fused_qat_indexer_scores(q, pooled, w, 128 ** -0.5), rtol=1e-5, atol=1e-5)


def test_fused_qat_indexer_scores_on_pool_rows_that_are_not_bf16_numbers():
    # the kernel multiplies on the bf16 matrix cores; pool values with more than 8 significant bits take
    # its exact three-piece form, tile by tile (here: mixed tiles, only rows 32..63 and the ragged tail carry
    # arbitrary float32 values)
    rng = np.random.default_rng(77)
    q, pooled, w = _score_inputs(131, rng)
    pooled = pooled.copy()
    pooled[0, 32:64] = rng.standard_normal((32, 128), dtype=np.float32)
    pooled[0, 128:] = rng.standard_normal((3, 128), dtype=np.float32) * 1e-3
    got = isk.fused_qat_indexer_scores(to_dev(q), to_dev(pooled), to_dev(w), 128 ** -0.5).cpu().numpy()
    want = ds4.fused_qat_indexer_scores(q, pooled, w, 128 ** -0.5)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    # integer pool values up to 2^20 and integer-valued lattice queries: every product and partial sum is an
    # exact float32 integer, so any lost piece would show
    qi = np.zeros((1, 4, 1, 128), dtype=np.float32)
    qi[0, :, 0, 0] = 1.0  # qat(e0) = H e0 / sqrt(128) per element: a constant row, checked through the oracle
    big = rng.integers(-(1 << 20), 1 << 20, (1, 70, 128)).astype(np.float32)
    wi = np.ones((1, 1, 4), dtype=np.float32)
    got = isk.fused_qat_indexer_scores(to_dev(qi), to_dev(big), to_dev(wi), 1.0).cpu().numpy()
    want = ds4.fused_qat_indexer_scores(qi, big, wi, 1.0)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=0)


def test_fused_scores_known_answer_ones():
    # qat(ones) = [12, 0, ...]: score = 144 / sqrt(128) per unit weight
    q = torch.ones((1, 2, 1, 128), device=dev())
    pooled = torch.zeros((1, 3, 128), device=dev())
    pooled[0, :, 0] = 12.0
    w = torch.tensor([[[1.0, 0.5]]], device=dev())
    got = isk.fused_qat_indexer_scores(q, pooled, w, 128 ** -0.5).cpu().numpy()
    np.testing.assert_allclose(got, np.full(3, 1.5 * 144.0 / np.sqrt(128.0)), rtol=1e-6)


@pytest.mark.parametrize("n_heads", [32, 48, 64])
@pytest.mark.parametrize("cap_valid", [(1024, 963), (1024, 1024), (963, 963), (33, 20)])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.float16, torch.bfloat16])
def test_fused_score_tail_bitexact(n_heads, cap_valid, wdtype):
    # reference :677-729
    capacity, valid = cap_valid
    rng = np.random.default_rng(100 + n_heads + capacity)
    raw = (rng.standard_normal((n_heads, capacity)) * 10.0 ** rng.integers(-8, 8, (n_heads, capacity))).astype(np.float32)
    w = (rng.standard_normal(n_heads) * 10.0 ** rng.integers(-3, 3, n_heads)).astype(np.float32)
    wt = to_dev(w.reshape(1, 1, n_heads), wdtype)
    params = torch.tensor([3844, valid], dtype=torch.int32, device=dev())
    got = isk.fused_score_tail(to_dev(raw.reshape(1, n_heads, 1, capacity)), wt, params, scale=128 ** -0.5)
    assert got.shape == (1, 1, capacity)
    want = ds4.score_tail(raw, wt.float().cpu().numpy().reshape(-1), np.array([3844, valid]), scale=128 ** -0.5)
    np.testing.assert_array_equal(bits(got.cpu().numpy().reshape(-1)), bits(want))


def test_fused_score_tail_special_values():
    # reference :731-750: -0, +-inf, NaN, denormals
    rng = np.random.default_rng(5)
    raw = rng.standard_normal((64, 40)).astype(np.float32)
    raw[0, 0] = -0.0
    raw[1, 1] = np.inf
    raw[2, 2] = -np.inf
    raw[3, 3] = np.nan
    raw[4, 4] = 1e-42
    raw[:, 5] = -1.0
    w = rng.standard_normal(64).astype(np.float32)
    params = torch.tensor([0, 40], dtype=torch.int32, device=dev())
    got = isk.fused_score_tail(to_dev(raw.reshape(1, 64, 1, 40)), to_dev(w.reshape(1, 1, 64)), params, scale=0.25)
    want = ds4.score_tail(raw, w, np.array([0, 40]), scale=0.25)
    g = got.cpu().numpy().reshape(-1)
    assert np.isnan(g[3]) and np.isnan(want[3])
    mask = ~np.isnan(want)
    np.testing.assert_array_equal(bits(g[mask]), bits(want[mask]))


@pytest.mark.parametrize("mag", [0.05, 1.0, 1.0e4, 1.0e-6, 0.0])
def test_fp8_kv_prefix_rows_bitexact(mag):
    # reference tests/test_deepseek_v4_decode_attention_kernel.py:144-181
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((37, 512)) * mag).astype(np.float32)
    got = dak.fp8_kv_prefix_rows(to_dev(x)).cpu().numpy()
    want = ds4.fp8_kv_roundtrip(x)
    np.testing.assert_array_equal(bits(got), bits(want))
    np.testing.assert_array_equal(got[:, 448:], x[:, 448:])


def test_fp8_kv_prefix_rows_exact_ties_take_lower_value():
    table = ds4.e4m3fn_values().astype(np.float64)
    mids = ((table[:-1] + table[1:]) / 2).astype(np.float32)   # 126 exact midpoints
    x = np.zeros((4, 512), dtype=np.float32)
    # block amax 448 -> scale 1, so values are their own normalised coordinates
    for r in range(4):
        x[r, 0:448:64] = 448.0
    x[0, 1:64] = mids[:63]
    x[1, 1:64] = -mids[63:126]
    x[2, 65:128] = mids[:63]
    x[3, 65:128] = table[1:64].astype(np.float32)       # exact table values stay
    got = dak.fp8_kv_prefix_rows(to_dev(x)).cpu().numpy()
    want = ds4.fp8_kv_roundtrip(x)
    np.testing.assert_array_equal(bits(got), bits(want))
    np.testing.assert_array_equal(got[0, 1:64], table[:63].astype(np.float32))
    np.testing.assert_array_equal(got[3, 65:128], x[3, 65:128])


def _yarn_inv_freq():
    return ds4.rope_inverse_frequencies(64, ds4.DS4_COMPRESS_ROPE_BASE, ds4.DS4_YARN).astype(np.float32)


def _prep_inputs(n_rows, seed, n_heads=64):
    # reference tests/test_deepseek_v4_decode_attention_kernel.py:40-62 (q here is any f16 row;
    # the reference ropes it first, which only changes the values)
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((n_heads, 128), dtype=np.float32).astype(np.float16)
    pooled = ds4.indexer_qat(rng.standard_normal((n_rows, 128), dtype=np.float32))
    w = (rng.standard_normal(n_heads, dtype=np.float32) * n_heads ** -0.5).astype(np.float32)
    kv_row = (rng.standard_normal(512, dtype=np.float32) * 0.05).astype(np.float16)
    return q, pooled, w, kv_row


@pytest.mark.parametrize("n_rows", [531, 961, 977, 40000])
def test_fused_decode_prep_scores_and_topk(n_rows):
    # reference :65-99: scores 1e-5, identical top-512 set
    q, pooled, w, kv_row = _prep_inputs(n_rows, 100 + n_rows)
    inv = _yarn_inv_freq()
    params = np.array([3844, 0], dtype=np.int32)
    sel, row, scores = dak.fused_decode_prep(to_dev(q), to_dev(pooled), to_dev(w), to_dev(kv_row), to_dev(inv),
                                             to_dev(params), scale=128 ** -0.5, topk=512)
    sel, row, scores = sel.cpu().numpy(), row.cpu().numpy(), scores.cpu().numpy()
    o_sel, o_row, o_scores = ds4.fused_decode_prep(q, pooled, w, kv_row, inv, params, scale=128 ** -0.5, topk=512)
    np.testing.assert_allclose(scores, o_scores, rtol=1e-5, atol=1e-5)
    # indices are bit-exact against the oracle's selection rule applied to the device's scores
    np.testing.assert_array_equal(sel, ds4.radix_select_topk(scores, 512))
    assert len(set(sel.tolist())) == 512
    # and equal the oracle's own selection as a set when its boundary is clear of the tolerance
    srt = np.sort(o_scores)[::-1]
    if srt[511] - srt[512] > 1e-4:
        assert set(sel.tolist()) == set(o_sel.tolist())
    np.testing.assert_array_equal(row.view(np.uint16), o_row.view(np.uint16))


@pytest.mark.parametrize("case", ["normal", "large", "tiny", "zeros"])
def test_fused_decode_prep_kv_row_bitexact(case):
    # reference :102-141
    rng = np.random.default_rng(7)
    mag = {"normal": 0.05, "large": 1.0e4, "tiny": 1.0e-6, "zeros": 0.0}[case]
    kv_row = (rng.standard_normal(512).astype(np.float32) * mag).astype(np.float16)
    q, pooled, w, _ = _prep_inputs(531, 8)
    inv = _yarn_inv_freq()
    for pos in (3844, 0, 1048575):
        params = np.array([pos, 0], dtype=np.int32)
        _, row, _ = dak.fused_decode_prep(to_dev(q), to_dev(pooled), to_dev(w), to_dev(kv_row), to_dev(inv),
                                          to_dev(params), scale=128 ** -0.5, topk=512)
        want = ds4.prepared_kv_row(kv_row, pos, inv)
        np.testing.assert_array_equal(row.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_fused_decode_prep_boundary_ties_take_lowest_rows():
    # reference :215-243: all pooled rows identical -> sel == arange(topk)
    rng = np.random.default_rng(3)
    q, _, w, kv_row = _prep_inputs(600, 3)
    one = ds4.indexer_qat(rng.standard_normal((1, 128), dtype=np.float32))
    pooled = np.repeat(one, 600, axis=0)
    sel, _, scores = dak.fused_decode_prep(to_dev(q), to_dev(pooled), to_dev(w), to_dev(kv_row),
                                           to_dev(_yarn_inv_freq()), to_dev(np.array([5, 0], np.int32)),
                                           scale=128 ** -0.5, topk=512)
    s = scores.cpu().numpy()
    assert np.all(s == s[0])
    np.testing.assert_array_equal(sel.cpu().numpy(), np.arange(512, dtype=np.int32))


def test_fused_decode_prep_integer_inputs_are_bitexact_end_to_end():
    # small-integer pool rows and a lattice query make every partial sum exact in float32, so
    # device scores equal the oracle's bit for bit (with many ties) and the indices must too
    rng = np.random.default_rng(17)
    n_rows = 3000
    q = ds4.hadamard128_unscaled(np.eye(128, dtype=np.float32)[:64] * 8.0)   # qat -> exact lattice rows
    pooled = rng.integers(-2, 3, (n_rows, 128)).astype(np.float32)
    w = (rng.integers(1, 5, 64) * 0.25).astype(np.float32)
    kv_row = np.zeros(512, dtype=np.float16)
    sel, _, scores = dak.fused_decode_prep(to_dev(q), to_dev(pooled), to_dev(w), to_dev(kv_row),
                                           to_dev(_yarn_inv_freq()), to_dev(np.array([0, 0], np.int32)),
                                           scale=0.25, topk=512)
    o_sel, _, o_scores = ds4.fused_decode_prep(q, pooled, w, kv_row, _yarn_inv_freq(), np.array([0, 0]),
                                               scale=0.25, topk=512)
    np.testing.assert_array_equal(bits(scores.cpu().numpy()), bits(o_scores.astype(np.float32)))
    np.testing.assert_array_equal(sel.cpu().numpy(), o_sel)


@pytest.mark.parametrize("shape_k", [((5,), 1), ((5,), 5), ((600,), 512), ((3, 977), 512), ((2, 8192), 2048),
                                     ((16, 32768), 2048), ((2, 70001), 2048), ((1, 32768), 32768),
                                     # rows of up to 2048 scores take a kernel of their own (one 256-thread workgroup
                                     # a row): its two widths, their boundaries, many rows, k = all rows
                                     ((70, 961), 512), ((9, 1024), 1024), ((5, 1025), 7), ((4, 2048), 2048),
                                     ((3, 2049), 100), ((300, 64), 33), ((130, 4096), 512), ((129, 7961), 512), ((128, 8192), 8000)])
def test_topk_select_bitexact(shape_k):
    shape, k = shape_k
    rng = np.random.default_rng(sum(shape) + k)
    cases = [rng.standard_normal(shape).astype(np.float32),                       # continuous
             (rng.integers(-3, 4, shape) * 0.5).astype(np.float32),               # heavy ties
             np.full(shape, 0.37, dtype=np.float32)]                              # all tie
    sp = rng.standard_normal(shape).astype(np.float32)
    flat = sp.reshape(-1)
    flat[rng.integers(0, flat.size, max(1, flat.size // 50))] = -0.0
    flat[rng.integers(0, flat.size, max(1, flat.size // 50))] = 0.0
    flat[rng.integers(0, flat.size, 3)] = np.inf
    flat[rng.integers(0, flat.size, 3)] = -np.inf
    flat[rng.integers(0, flat.size, 3)] = np.nan
    cases.append(sp)
    for s in cases:
        got = isk.topk_select(to_dev(s), k).cpu().numpy()
        assert got.shape == shape[:-1] + (k,) and got.dtype == np.int32
        rows = s.reshape(-1, shape[-1])
        g2 = got.reshape(-1, k)
        for b in range(rows.shape[0]):
            np.testing.assert_array_equal(g2[b], ds4.radix_select_topk(rows[b], k))


@pytest.mark.parametrize("n_k", [(32768, 2048), (32768, 512), (20000, 2048), (8192, 2048), (8192, 64), (3000, 1)])
def test_topk_select_sample_misleads(n_k):
    """The kernel guesses a pivot from every C-th row (C = 8 up to 8192 rows, 32 up to 32768) and must
    fall back to the full select when the guess is bad: rows whose sampled positions are all small, all
    large, or all equal must still give the exact answer."""
    n, k = n_k
    c = 8 if n <= 8192 else 32
    rng = np.random.default_rng(n + k)
    base = rng.standard_normal((4, n)).astype(np.float32)
    lo = base.copy()
    lo[:, ::c] = -50.0 - rng.random((4, len(range(0, n, c)))).astype(np.float32)   # pivot far too low
    hi = base.copy()
    hi[:, ::c] = 50.0 + rng.random((4, len(range(0, n, c)))).astype(np.float32)    # pivot far too high
    eq = base.copy()
    eq[:, ::c] = 0.25                                                              # one value in the sample
    few = np.zeros((4, n), dtype=np.float32)                                       # k-th key inside a huge tie
    few[:, rng.integers(0, n, max(1, k // 2))] = 1.0
    edge = base.copy()                                                             # exactly k rows above the rest
    edge[:, :] = -1.0
    edge[:, rng.choice(n, k, replace=False)] = rng.random(k).astype(np.float32) + 1.0
    for s in (lo, hi, eq, few, edge):
        got = isk.topk_select(to_dev(s), k).cpu().numpy()
        for b in range(s.shape[0]):
            np.testing.assert_array_equal(got[b], ds4.radix_select_topk(s[b], k))


def test_validation_messages_match_reference():
    # reference :125-133, :211-238, :752-776 (rejections happen before any device work)
    z = torch.zeros
    with pytest.raises(ValueError, match="128-wide"):
        isk.indexer_qat_rows(z((4, 64)))
    with pytest.raises(ValueError, match="float32, float16, or bfloat16"):
        isk.indexer_qat_rows(z((4, 128), dtype=torch.int32))
    with pytest.raises(ValueError, match="one decode token"):
        isk.fused_qat_indexer_scores(z((2, 64, 1, 128)), z((1, 8, 128)), z((1, 1, 64)), 1.0)
    with pytest.raises(ValueError, match="head_dim=128"):
        isk.fused_qat_indexer_scores(z((1, 64, 1, 64)), z((1, 8, 64)), z((1, 1, 64)), 1.0)
    with pytest.raises(ValueError, match="between 1 and 64 heads"):
        isk.fused_qat_indexer_scores(z((1, 65, 1, 128)), z((1, 8, 128)), z((1, 1, 65)), 1.0)
    with pytest.raises(ValueError, match="pooled_qat and weights must be float32"):
        isk.fused_qat_indexer_scores(z((1, 64, 1, 128)), z((1, 8, 128), dtype=torch.float16), z((1, 1, 64)), 1.0)
    with pytest.raises(RuntimeError, match="HIP device"):
        isk.indexer_qat_rows(z((4, 128)))
