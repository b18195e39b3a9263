"""Pins for the DeepSeek-V4 half of the CPU oracle (no GPU needed).

Each test checks an oracle function against something the oracle did not
produce: a known-answer value held by the reference's own tests (cited), a
closed form, a library routine, or brute force on small inputs.
"""

import math

import numpy as np
import pytest
import scipy.linalg
import torch

from oracle import ds4


# ---------------------------------------------------------------- Hadamard / QAT

def test_hadamard128_matches_sylvester_matrix_and_is_involutive():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((7, 128)).astype(np.float32)
    H = scipy.linalg.hadamard(128).astype(np.float64)
    want = x.astype(np.float64) @ H.T
    got = ds4.hadamard128_unscaled(x)
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-5)
    twice = ds4.hadamard128_unscaled(got)
    np.testing.assert_allclose(twice, 128.0 * x, rtol=0, atol=2e-3)
    # one-hot rows pick single columns of H: catches a wrong stride order or sign
    eye = np.eye(128, dtype=np.float32)
    np.testing.assert_array_equal(ds4.hadamard128_unscaled(eye), H.T.astype(np.float32))


def test_qat_of_ones_is_twelve_then_zeros():
    # reference KAT: tests/test_deepseek_v4_model.py:1064-1070 (score 144/sqrt(128))
    out = ds4.indexer_qat(np.ones((1, 128), dtype=np.float32))
    want = np.zeros((1, 128), dtype=np.float32)
    want[0, 0] = 12.0
    np.testing.assert_array_equal(out, want)
    score = ds4.indexer_scores_f64(out, out, np.ones(1), 128 ** -0.5)
    assert math.isclose(score[0], 144.0 / math.sqrt(128.0), rel_tol=1e-12)


def test_qat_lattice_invariants_and_tie_rule():
    rng = np.random.default_rng(1234)
    y = rng.standard_normal((64, 128)).astype(np.float32)
    out = ds4.indexer_fp4_act_roundtrip(y)
    g = np.abs(y.reshape(64, 4, 32))
    amax = g.max(-1, keepdims=True)
    # exact power of two scale: smallest 2^k with amax/6 <= 2^k
    k = np.ceil(np.log2(amax.astype(np.float64) / 6.0))
    scale = np.exp2(k)
    ratio = np.abs(out.reshape(64, 4, 32).astype(np.float64)) / scale
    lattice = set(ds4.E2M1_LATTICE.tolist())
    assert set(np.unique(ratio).tolist()) <= lattice
    # error bound: half the widest lattice gap (2.0) times the scale
    err = np.abs(out.reshape(64, 4, 32) - y.reshape(64, 4, 32))
    assert np.all(err <= 1.0 * scale + 1e-6)
    # idempotent on rows already on the lattice
    np.testing.assert_array_equal(ds4.indexer_fp4_act_roundtrip(out), out)
    # zeros stay zeros, and signed zero input gives zeros
    z = np.zeros((1, 128), dtype=np.float32)
    np.testing.assert_array_equal(ds4.indexer_fp4_act_roundtrip(z), z)
    # exact midpoints go to the LOWER lattice value (first-wins argmin);
    # group amax 6 -> scale 1 so values are the lattice coordinates themselves
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
    lows = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0], dtype=np.float32)
    row = np.zeros((1, 128), dtype=np.float32)
    row[0, 0] = 6.0
    row[0, 1:8] = mids
    row[0, 8:15] = -mids
    got = ds4.indexer_fp4_act_roundtrip(row)
    np.testing.assert_array_equal(got[0, 1:8], lows)
    np.testing.assert_array_equal(got[0, 8:15], -lows)
    assert got[0, 0] == 6.0


def test_pow2_group_scale_is_exact_power_of_two_for_ordinary_exponents():
    # exp(k*ln2f) in float32 is exactly 2^k for |k| <= 12 and a few ulp off
    # beyond (the reference keeps those bits: indexer_score_kernel.py:21-26)
    for denom in (6.0, 448.0):
        for k in range(-30, 31):
            for frac in (0.5000001, 0.75, 0.9999999, 1.0):
                amax = np.float32(denom * frac * 2.0 ** k)
                got = float(ds4.pow2_group_scale(np.asarray([amax]), denom)[0])
                r = float(np.float32(amax) / np.float32(denom))
                kk = math.ceil(math.log2(r))
                if frac in (1.0, 0.5000001):
                    # within an ulp of a power of two the float32 log/ln2
                    # quotient may land on either side of the integer
                    cands = (kk - 1, kk, kk + 1)
                else:
                    cands = (kk,)
                ok = False
                for c in cands:
                    want = 2.0 ** c
                    if abs(c) <= 12:
                        ok = ok or got == want
                    else:
                        ok = ok or abs(got / want - 1.0) < 4e-6
                assert ok, (denom, k, frac, got)
    # the amax floor keeps the smallest scale near 2^-126 and tiny rows quantise to zero
    out = ds4.indexer_fp4_act_roundtrip(np.full((1, 32), 1e-45, dtype=np.float32))
    assert np.all(out == 0.0)


# ---------------------------------------------------------------- E4M3FN

def test_e4m3fn_table_matches_torch_float8_decode():
    codes = torch.arange(127, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    np.testing.assert_array_equal(ds4.e4m3fn_values(), want)
    allc = np.arange(256, dtype=np.uint8)
    want_all = torch.from_numpy(allc).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    np.testing.assert_array_equal(ds4.e4m3_decode(allc), want_all)


def test_e4m3_encode_matches_torch_cast():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(20000) * np.exp(rng.uniform(-8, 6, 20000))).astype(np.float32)
    x = np.clip(x, -448, 448)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = ds4.e4m3_encode(x)
    # -0 vs +0 codes may differ on tiny negatives; compare decoded values
    np.testing.assert_array_equal(ds4.e4m3_decode(got), ds4.e4m3_decode(want))


def test_fp8_kv_roundtrip_matches_torch_cast_away_from_ties():
    rng = np.random.default_rng(7)
    for mag in (0.05, 1.0, 1.0e4, 1.0e-6):
        x = (rng.standard_normal((16, 512)) * mag).astype(np.float32)
        got = ds4.fp8_kv_roundtrip(x)
        np.testing.assert_array_equal(got[:, 448:], x[:, 448:])
        blocks = x[:, :448].reshape(16, 7, 64)
        amax = np.maximum(np.abs(blocks).max(-1, keepdims=True), np.float32(1e-4)).astype(np.float64)
        scale = np.exp2(np.ceil(np.log2(amax / 448.0)))
        n = (blocks / scale).astype(np.float32)
        q = torch.from_numpy(n).to(torch.float8_e4m3fn).to(torch.float32).numpy()
        want = (q * scale).astype(np.float32).reshape(16, 448)
        # torch rounds exact midpoints to even, the reference takes the lower
        # value; random float32 data does not hit exact midpoints
        if mag == 1.0e-6:
            # block scale 2^-22: exp(k*ln2f) is a few float32 ulp off 2^k there
            np.testing.assert_allclose(got[:, :448], want, rtol=4e-6, atol=0)
        else:
            np.testing.assert_array_equal(got[:, :448], want)
    z = np.zeros((2, 512), dtype=np.float32)
    np.testing.assert_array_equal(ds4.fp8_kv_roundtrip(z), z)


def test_fp8_nearest_takes_lower_value_on_exact_midpoints():
    table = ds4.e4m3fn_values().astype(np.float64)
    mids = ((table[:-1] + table[1:]) / 2).astype(np.float32)
    got = ds4.fp8_nearest_first_wins(mids)
    np.testing.assert_array_equal(got, table[:-1].astype(np.float32))


# ---------------------------------------------------------------- scores / tail

def test_indexer_scores_known_answers():
    # reference KAT tests/test_deepseek_v4_attention.py:197-200: 64 heads of ones -> 64*scale
    scale = ds4.indexer_weight_scale(128, 64)
    assert math.isclose(scale, (128 ** -0.5) * (64 ** -0.5))
    raw = np.ones((1, 64, 1))
    w = np.ones((1, 64))
    np.testing.assert_allclose(ds4.indexer_weighted_scores(raw, w), [[64.0 * scale]])
    # relu drops negative heads; weights may be negative
    q = np.zeros((2, 128), dtype=np.float32)
    q[0, 0] = 1.0
    q[1, 0] = -1.0
    p = np.zeros((1, 128), dtype=np.float32)
    p[0, 0] = 3.0
    got = ds4.indexer_scores_f64(q, p, np.array([2.0, 5.0]), 0.5)
    np.testing.assert_allclose(got, [3.0 * 0.5 * 2.0])


def test_score_tail_value_pad_and_special_values():
    rng = np.random.default_rng(164)
    H, C, valid = 64, 33, 20
    raw = (rng.standard_normal((H, C)) * 10.0 ** rng.integers(-8, 8, (H, C))).astype(np.float32)
    w = (rng.standard_normal(H) * 10.0 ** rng.integers(-3, 3, H)).astype(np.float32)
    neg = ds4.score_tail(raw, w, np.array([3844, valid], dtype=np.int32), scale=128 ** -0.5)
    want = -(np.maximum(raw.astype(np.float64), 0) * (128 ** -0.5)
             * (w.astype(np.float64) * 64 ** -0.5)[:, None]).sum(0)
    np.testing.assert_allclose(neg[:valid], want[:valid], rtol=2e-5, atol=0)
    assert np.all(np.isposinf(neg[valid:]))
    # special values: NaN passes through relu, -inf and -0 clamp to +0, +inf stays
    raw2 = np.zeros((32, 4), dtype=np.float32)
    raw2[0, 0] = np.nan
    raw2[0, 1] = -np.inf
    raw2[0, 2] = np.inf
    raw2[0, 3] = -0.0
    neg2 = ds4.score_tail(raw2, np.ones(32, dtype=np.float32), np.array([0, 4], dtype=np.int32), scale=1.0)
    assert np.isnan(neg2[0])
    assert neg2[1] == 0.0 and np.signbit(neg2[1])      # -(+0.0)
    assert np.isneginf(neg2[2])
    assert neg2[3] == 0.0 and np.signbit(neg2[3])


def test_pad_scores_and_params():
    np.testing.assert_array_equal(ds4.decode_step_params(3844, 961), np.array([3844, 961], np.int32))
    s = ds4.pad_scores_to_capacity(np.ones((1, 1, 8), np.float32), 5)
    assert np.all(s[..., :5] == 1) and np.all(np.isneginf(s[..., 5:]))


# ---------------------------------------------------------------- top-k

def test_causal_topk_reference_known_answer():
    # reference KAT tests/test_deepseek_v4_attention.py:203-244
    pool = np.array([0, 1, 2, 3], dtype=np.int64)
    raw = np.array([[[1.0, 20.0, 1000.0, 1000.0], [2.0, 10.0, 1000.0, 1000.0]],
                    [[1.0, 9.0, 1000.0, 1000.0], [2.0, 8.0, 1000.0, 1000.0]]])
    topk = ds4.causal_indexer_topk(raw, np.ones((2, 2)), np.array([3, 7]), pool, 4,
                                   topk=3, index_head_dim=128, n_heads=2)
    np.testing.assert_array_equal(topk, [[0, -1, -1], [1, 0, -1]])


def test_radix_select_matches_bruteforce_and_tie_rule():
    rng = np.random.default_rng(3)
    for n, k in [(5, 1), (5, 5), (600, 512), (977, 512), (4096, 2048), (70000, 2048)]:
        # heavy ties: few distinct values
        s = rng.integers(-3, 4, n).astype(np.float32) * 0.5
        got = ds4.radix_select_topk(s, k)
        brute = ds4.topk_lexsort(s, k)
        assert sorted(got.tolist()) == sorted(brute.tolist())
        # emission order: strictly-above ascending, then ties ascending
        thr = np.sort(s)[::-1][k - 1]
        above = np.flatnonzero(s > thr)
        ties = np.flatnonzero(s == thr)[:k - above.size]
        np.testing.assert_array_equal(got, np.concatenate([above, ties]))
        # continuous scores: equals argpartition as a set
        c = rng.standard_normal(n).astype(np.float32)
        got = ds4.radix_select_topk(c, k)
        assert set(got.tolist()) == set(np.argpartition(-c, k - 1)[:k].tolist())
    # all-tie -> arange (reference test_deepseek_v4_decode_attention_kernel.py:215-243)
    np.testing.assert_array_equal(ds4.radix_select_topk(np.full(600, 0.37, np.float32), 512),
                                  np.arange(512))


def test_score_key_total_order_on_special_values():
    vals = np.array([-np.inf, -1.0, -1e-45, -0.0, 0.0, 1e-45, 1.0, np.inf, np.nan], dtype=np.float32)
    keys = ds4.score_key(vals).astype(np.int64)
    assert np.all(np.diff(keys) > 0)   # -0.0 < +0.0 and +NaN above +inf
    s = np.array([0.0, -0.0, 0.0, -0.0], dtype=np.float32)
    np.testing.assert_array_equal(ds4.radix_select_topk(s, 3), [0, 2, 1])


# ---------------------------------------------------------------- rope

def test_yarn_inverse_frequencies_and_angles_pinned():
    # values held by the reference: tests/test_deepseek_v4_attention.py:56-122
    freqs = ds4.rope_inverse_frequencies(64, ds4.DS4_COMPRESS_ROPE_BASE, ds4.DS4_YARN)
    np.testing.assert_allclose(freqs[[0, 8, 16, 24, 31]],
                               [1.0, 5.0e-2, 2.265625e-3, 1.953125e-5, 5.68052903691e-7],
                               rtol=0, atol=1e-14)
    ang = ds4.rope_angles([65535, 131072, 1048575], base=ds4.DS4_COMPRESS_ROPE_BASE, yarn=ds4.DS4_YARN)
    np.testing.assert_allclose(
        ang[:, [0, 8, 16, 24, 31]],
        [[65535.0, 3276.75, 148.477734375, 1.27998046875, 0.0372273470],
         [131072.0, 6553.6, 296.96, 2.56, 0.0744558302],
         [1048575.0, 52428.75, 2375.677734375, 20.47998046875, 0.595646073]],
        rtol=0, atol=1e-9)
    swa = ds4.rope_inverse_frequencies(64, ds4.DS4_SWA_ROPE_BASE, None)
    assert math.isclose(swa[16], 1.0e-2)
    swa_ang = ds4.rope_angles([131071, 1048575], base=ds4.DS4_SWA_ROPE_BASE)
    np.testing.assert_allclose(swa_ang[:, [8, 31]], [[13107.1, 17.4785987635], [104857.5, 139.829723573]],
                               rtol=0, atol=1e-9)


def test_rope_tail_rotates_only_tail_and_inverse_cancels():
    # reference tests/test_deepseek_v4_attention.py:125-143
    rng = np.random.default_rng(0)
    x = rng.normal(size=(2, 512)).astype(np.float32)
    pos = np.array([5, 65536])
    rot = ds4.apply_rope_tail(x, pos, base=ds4.DS4_COMPRESS_ROPE_BASE, yarn=ds4.DS4_YARN)
    np.testing.assert_array_equal(rot[:, :448], x[:, :448])
    assert not np.allclose(rot[:, -64:], x[:, -64:])
    back = ds4.apply_rope_tail(rot, pos, base=ds4.DS4_COMPRESS_ROPE_BASE, yarn=ds4.DS4_YARN, inverse=True)
    np.testing.assert_allclose(back, x, rtol=2e-6, atol=2e-6)
    # a pair (1, 0) at angle theta becomes (cos, sin): pins pair layout and sign
    one = np.zeros((1, 512))
    one[0, 448] = 1.0
    r = ds4.apply_rope_tail(one, [3], base=10000.0)
    assert math.isclose(r[0, 448], math.cos(3.0)) and math.isclose(r[0, 449], math.sin(3.0))


def test_lowp_rope_tracks_float64_rope():
    rng = np.random.default_rng(11)
    inv = ds4.rope_inverse_frequencies(64, ds4.DS4_COMPRESS_ROPE_BASE, ds4.DS4_YARN).astype(np.float32)
    x = ds4.round_f16(rng.standard_normal((3, 512)).astype(np.float32) * 0.5)
    got = ds4.partial_rope_lowp(x, 3844, inv)
    want = ds4.apply_rope_tail(x.astype(np.float64), [3844] * 3, base=ds4.DS4_COMPRESS_ROPE_BASE,
                               yarn=ds4.DS4_YARN)
    np.testing.assert_array_equal(got[:, :448], x[:, :448])
    np.testing.assert_allclose(got, want, rtol=0, atol=4e-3)
    back = ds4.partial_rope_lowp(got, 3844, inv, inverse=True)
    np.testing.assert_allclose(back, x, rtol=0, atol=6e-3)


# ---------------------------------------------------------------- attention

_YARN = {"factor": 16.0, "original_seq_len": 65536, "beta_fast": 32, "beta_slow": 1}


def test_fused_partial_rope_float32_tracks_float64_rope_and_copies_the_head():
    # pins: the float64 closed form of attention.py:117-156; leading channels and signed zeros untouched
    rng = np.random.default_rng(5)
    x = (2.0 * rng.standard_normal((2, 5, 7, 128))).astype(np.float32)
    x[0, 0, 0, :4] = -0.0
    inv = ds4.rope_inverse_frequencies(64, 160000.0, _YARN).astype(np.float32)
    for offset, inverse in ((0, False), (3855, True)):
        got = ds4.fused_partial_rope(x, inv, offset=offset, inverse=inverse)
        want = ds4.apply_rope_tail(x.astype(np.float64), np.arange(offset, offset + 7), base=160000.0, yarn=_YARN,
                                   inverse=inverse)
        np.testing.assert_array_equal(got[..., :64].view(np.uint32), x[..., :64].view(np.uint32))
        # float32 angles lose about |theta| * 2^-24: a few 1e-4 at position 3855 on values up to ~8
        assert np.abs(got - want).max() < (2e-5 if offset == 0 else 4e-3)
    # offset form == positions form on the same positions; inverse undoes forward
    pos = np.arange(40, 47, dtype=np.float32)
    a = ds4.fused_partial_rope(x, inv, offset=40)
    b = ds4.fused_partial_rope(x, inv, positions=pos)
    np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))
    back = ds4.fused_partial_rope(a, inv, offset=40, inverse=True)
    assert np.abs(back - x).max() < 2e-6 * 8


def test_fused_partial_rope_16bit_rounds_every_operation():
    # pin: the same rotation carried out in NumPy's native float16 arithmetic, which rounds each
    # product and sum to float16 by construction
    rng = np.random.default_rng(6)
    x16 = (2.0 * rng.standard_normal((3, 4, 512))).astype(np.float16)
    inv = ds4.rope_inverse_frequencies(64, 10000.0).astype(np.float32)
    offset = 17
    got = ds4.fused_partial_rope(x16.astype(np.float32), inv, offset=offset, dtype="float16")
    want = x16.copy()
    for l in range(4):
        theta = (np.float32(offset + l) * inv).astype(np.float32)
        c = np.cos(theta.astype(np.float64)).astype(np.float32).astype(np.float16)
        s = np.sin(theta.astype(np.float64)).astype(np.float32).astype(np.float16)
        x0, x1 = x16[:, l, 448::2], x16[:, l, 449::2]
        want[:, l, 448::2] = x0 * c - x1 * s
        want[:, l, 449::2] = x0 * s + x1 * c
    np.testing.assert_array_equal(got.astype(np.float16).view(np.uint16), want.view(np.uint16))
    # bfloat16: results are bfloat16 values and stay within one bfloat16 step of the float32 rotation
    xb = ds4.round_bf16((2.0 * rng.standard_normal((2, 3, 128))).astype(np.float32))
    gb = ds4.fused_partial_rope(xb, inv, offset=3, dtype="bfloat16")
    np.testing.assert_array_equal(gb.view(np.uint32), ds4.round_bf16(gb).view(np.uint32))
    g32 = ds4.fused_partial_rope(xb, inv, offset=3)
    assert np.abs(gb - g32).max() <= 2.0 ** -7 * np.abs(g32).max()


def test_sink_attention_known_answer_and_softmax_limit():
    # reference tests/test_deepseek_v4_attention.py:146-160
    scores = np.array([[0.25]])
    values = np.array([[[8.0, -4.0]]])
    out = ds4.sink_softmax_attention(scores, values, np.array([1.25]))
    den = math.exp(0.25 - 1.25) + 1.0
    np.testing.assert_allclose(out, values[:, 0, :] * (math.exp(-1.0) / den))
    # sink = -inf reduces to the library softmax
    rng = np.random.default_rng(2)
    s = rng.standard_normal((4, 9))
    v = rng.standard_normal((9, 5))
    got = ds4.sink_softmax_attention(s, v[None], np.full(4, -np.inf))
    want = torch.softmax(torch.from_numpy(s), -1).numpy() @ v
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


def test_visibility_known_answers():
    # reference tests/test_deepseek_v4_attention.py:163-189
    vis4 = ds4.compressed_visibility([2, 3, 4, 127, 128], np.arange(34), 4)
    assert not vis4[0, 0] and vis4[1, 0] and vis4[2, 0]
    assert vis4[3, 31] and not vis4[3, 32] and vis4[4, 31] and not vis4[4, 32]
    np.testing.assert_array_equal(ds4.visible_compressed_count([3, 4, 65535, 65536, 1048575], 4),
                                  [1, 1, 16384, 16384, 262144])
    np.testing.assert_array_equal(ds4.compressed_rope_positions([0, 1, 8191], 128), [0, 128, 1048448])


def test_visit_rows_rules():
    # full ring, window smaller than ring, circular start
    raw, comp = ds4.indexed_visit_rows(raw_cap=9, n_comp=32, topk=np.arange(16), qpos=136, last_pos=136,
                                       window=128, ratio=4, raw_start=0)
    assert raw == list(range(9)) and comp == list(range(16))
    raw, _ = ds4.indexed_visit_rows(raw_cap=8, n_comp=4, topk=[], qpos=20, last_pos=20,
                                    window=3, ratio=4, raw_start=5)
    # positions 18,19,20 are logical rows 5,6,7 -> physical (5+5)%8, (5+6)%8, (5+7)%8
    assert raw == [2, 3, 4]
    # negative ids skipped, first id >= visible stops the walk (later valid ids dropped)
    _, comp = ds4.indexed_visit_rows(raw_cap=1, n_comp=100, topk=[3, -1, 2, 9, 1], qpos=19, last_pos=19,
                                     window=128, ratio=4, raw_start=0)
    assert comp == [3, 2]            # visible = 20//4 = 5; 9 >= 5 stops before 1
    # ratio 0 means the whole pool is visible
    _, comp = ds4.indexed_visit_rows(raw_cap=1, n_comp=6, topk=[5, 4], qpos=0, last_pos=0,
                                     window=128, ratio=0, raw_start=0)
    assert comp == [5, 4]


def test_indexed_decode_equals_selected_rows_reference_when_all_visible():
    # the reference's own parity test shape: test_deepseek_v4_indexed_attention_kernel.py:61-89
    rng = np.random.default_rng(123)
    q = rng.standard_normal((8, 512)).astype(np.float32)
    raw = rng.standard_normal((9, 512)).astype(np.float16)
    comp = rng.standard_normal((32, 512)).astype(np.float16)
    topk = np.arange(16, dtype=np.int32)
    sinks = rng.standard_normal(8).astype(np.float32)
    a = ds4.indexed_mixed_attention_decode(q, raw, comp, topk, sinks, pos0=136)
    b = ds4.selected_rows_attention_reference(q, raw, comp, topk, sinks)
    np.testing.assert_allclose(a, b, rtol=2e-3, atol=2e-3)
    # against torch softmax with the sink as an extra zero-value key
    qh = q.astype(np.float16).astype(np.float64)
    rows = np.concatenate([raw, comp[:16]]).astype(np.float64)
    s = torch.from_numpy(np.concatenate([qh @ rows.T * 512 ** -0.5, sinks[:, None].astype(np.float64)], 1))
    p = torch.softmax(s, -1).numpy()[:, :-1]
    np.testing.assert_allclose(a, p @ rows, rtol=1e-10, atol=1e-10)


def test_fused_decode_sdpa_without_rope_reduces_to_plain_attention():
    rng = np.random.default_rng(21)
    q = (0.1 * rng.standard_normal((4, 512))).astype(np.float16)
    window = (0.1 * rng.standard_normal((6, 512))).astype(np.float16)
    row = (0.1 * rng.standard_normal(512)).astype(np.float16)
    pooled = (0.1 * rng.standard_normal((20, 512))).astype(np.float16)
    sel = np.array([3, 7, 11], dtype=np.int32)
    sinks = rng.standard_normal(4).astype(np.float16)
    inv0 = np.zeros(32, dtype=np.float32)          # theta = 0: rope is the identity
    out = ds4.fused_decode_sdpa(q, window, row, pooled, sel, sinks, inv0, np.array([77, 2]), scale=512 ** -0.5)
    win = window.copy()
    win[2] = row
    keys = np.concatenate([win, pooled[sel]]).astype(np.float64)
    want = ds4.attend_rows_f64(q.astype(np.float64), keys, sinks.astype(np.float64), 512 ** -0.5)
    np.testing.assert_allclose(out.astype(np.float64), want, rtol=0, atol=1e-3)


def test_prepared_kv_row_parts():
    rng = np.random.default_rng(7)
    inv = ds4.rope_inverse_frequencies(64, ds4.DS4_COMPRESS_ROPE_BASE, ds4.DS4_YARN).astype(np.float32)
    row = (rng.standard_normal(512) * 0.05).astype(np.float16)
    got = ds4.prepared_kv_row(row, 3844, inv)
    assert got.dtype == np.float16
    want_tail = ds4.apply_rope_tail(row.astype(np.float64).reshape(1, 512), [3844],
                                    base=ds4.DS4_COMPRESS_ROPE_BASE, yarn=ds4.DS4_YARN)[0, 448:]
    np.testing.assert_allclose(got[448:].astype(np.float64), want_tail, rtol=0, atol=3e-4)
    # prefix: relative fp8 error bound 2^-4 of the block scale grid
    err = np.abs(got[:448].astype(np.float64) - row[:448].astype(np.float64))
    amax = np.abs(row[:448].astype(np.float64)).reshape(7, 64).max(-1)
    assert np.all(err.reshape(7, 64) <= amax[:, None] * 2.0 ** -3)


def test_sparse_mla_and_fp8_indexer_closed_forms():
    rng = np.random.default_rng(9)
    q = rng.standard_normal((2, 4, 576))
    kv = rng.standard_normal((2, 50, 576))
    rows = np.stack([rng.permutation(50)[:20], rng.permutation(50)[:20]])
    rows[1, 3] = -1
    out = ds4.sparse_mla_decode(q, kv, rows, scale=576 ** -0.5)
    for b in range(2):
        r = rows[b][rows[b] >= 0]
        s = torch.from_numpy(q[b] @ kv[b][r].T * 576 ** -0.5)
        want = torch.softmax(s, -1).numpy() @ kv[b][r][:, :512]
        np.testing.assert_allclose(out[b], want, rtol=1e-10, atol=1e-12)
    codes = rng.integers(0, 256, (1, 7, 128)).astype(np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0
    ks = rng.uniform(0.5, 2.0, (1, 7)).astype(np.float32)
    qi = rng.standard_normal((1, 3, 128)).astype(np.float32)
    w = rng.uniform(0, 1, (1, 3)).astype(np.float32)
    got = ds4.indexer_scores_fp8(qi, codes, ks, w)
    k = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float64).numpy() * ks[..., None]
    want = (np.maximum(np.einsum("bhd,bnd->bhn", qi.astype(np.float64), k), 0) * w[..., None]).sum(1)
    np.testing.assert_allclose(got, want, rtol=1e-12)


def test_live_qat_matches_a1_off_midpoints_and_prefers_even_on_ties():
    """indexed_attention_kernel.py:1137-1141: the live QAT differs from a1 only on exact midpoints
    (even lattice index wins) and where exp(k ln2) is not exactly 2^k."""
    rng = np.random.default_rng(11)
    x = rng.standard_normal((64, 128)).astype(np.float32)
    a1, live = ds4.indexer_qat(x), ds4.indexer_q_qat_live(x)
    np.testing.assert_allclose(live, a1, rtol=1e-5, atol=1e-5)  # the reference test's own bar
    mid = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)  # the seven lattice midpoints
    np.testing.assert_array_equal(ds4.e2m1_nearest_prefer_even(mid),
                                  np.array([0.0, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0], dtype=np.float32))
    # off the midpoints it is plain nearest
    np.testing.assert_array_equal(ds4.e2m1_nearest_prefer_even(np.array([0.2, 0.3, 1.6, 2.6, 5.1, 6.0], dtype=np.float32)),
                                  np.array([0.0, 0.5, 1.5, 3.0, 6.0, 6.0], dtype=np.float32))
    # a row whose groups have amax exactly 6 * 2^k after the Hadamard scale cannot be built exactly
    # (the scale constant is not 2^-3.5), so the scale rule is pinned on its own: exact powers of two
    x = np.array([1.0, 1.0000001, 0.5, 0.49999997, 2.0, 3.0, 2.0 ** -100, 1.5 * 2.0 ** -100], dtype=np.float32)
    np.testing.assert_array_equal(ds4.exp2_ceil_log2(x),
                                  np.array([1.0, 2.0, 0.5, 0.5, 2.0, 4.0, 2.0 ** -100, 2.0 ** -99], dtype=np.float32))


def test_tiled_live_scores_closed_form_and_visibility():
    rng = np.random.default_rng(12)
    B, H, T, P = 2, 8, 5, 9
    q = rng.standard_normal((B, H, T, 128)).astype(np.float32)
    comp = rng.standard_normal((B, P, 128)).astype(np.float32)
    w = rng.uniform(0, 1, (B, T, H)).astype(np.float32)
    got = ds4.indexer_scores_tiled_live(q, w, comp, pos0=6, ratio=4)
    qh, ch = q.astype(np.float16).astype(np.float64), comp.astype(np.float16).astype(np.float64)
    for b in range(B):
        for t in range(T):
            visible = min(P, (6 + t + 1) // 4)
            for c in range(P):
                want = sum(max(float(qh[b, h, t] @ ch[b, c]), 0.0) * float(w[b, t, h]) for h in range(H))
                if c < visible:
                    assert abs(got[b, t, c] - want) < 1e-9
                else:
                    assert got[b, t, c] == -np.inf


def test_round_bf16_and_f16_match_torch_casts():
    # a truncating or round-half-up restatement would pass idempotence; the library cast pins the rule
    rng = np.random.default_rng(8)
    x = rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 20000).astype(np.float32)
    ties = (np.arange(1, 4097, dtype=np.uint32) << 16 | 0x8000).view(np.float32)          # exact bf16 midpoints
    special = np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-40, 3.3895314e38, 65504.0, 65520.0, 65519.99],
                       dtype=np.float32)
    for a in (x, ties, -ties, special):
        want = torch.from_numpy(a).to(torch.bfloat16).to(torch.float32).numpy()
        np.testing.assert_array_equal(ds4.round_bf16(a).view(np.uint32), want.view(np.uint32))
        want16 = torch.from_numpy(a).to(torch.float16).to(torch.float32).numpy()
        np.testing.assert_array_equal(ds4.round_f16(a).view(np.uint32), want16.view(np.uint32))
    assert np.isnan(ds4.round_bf16(np.array([np.nan], np.float32))).all()


def _walk_token(raw, comp, ids, qpos, newest_pos, window, ratio, raw_start):
    """Rows one query visits, by absolute position (independent of ds4.indexed_visit_rows): the ring holds
    the raw_cap newest positions ending at newest_pos, position p at row (raw_start + p - oldest) % raw_cap."""
    raw_cap = raw.shape[0]
    oldest = newest_pos - raw_cap + 1
    rows = []
    for p in range(max(0, oldest), newest_pos + 1):
        if p > qpos or (window and p <= qpos - window):
            continue
        rows.append(raw[(raw_start + p - oldest) % raw_cap])
    visible = comp.shape[0] if ratio == 0 else min((qpos + 1) // ratio, comp.shape[0])
    for i in ids:
        if i < 0:
            continue
        if i >= visible:
            break
        rows.append(comp[i])
    return np.stack(rows) if rows else np.zeros((0, raw.shape[1]), np.float32)


def test_indexed_prefill_against_an_independent_walk_and_the_composed_reference_form():
    rng = np.random.default_rng(77)
    T, H, P = 37, 4, 30
    q = (rng.standard_normal((T, H, 512)) * 0.4).astype(np.float32)
    comp = (rng.standard_normal((P, 512)) * 0.5).astype(np.float16)
    sinks = rng.standard_normal(H).astype(np.float32)
    for pos0, raw_cap, window, raw_start, ratio in ((0, 37, 16, 0, 4), (50, 37, 128, 11, 4), (3, 64, 8, 63, 4),
                                                    (90, 20, 0, 5, 0)):
        raw = (rng.standard_normal((raw_cap, 512)) * 0.5).astype(np.float16)
        ids = np.stack([np.sort(rng.choice(P, 9, replace=False)) for _ in range(T)]).astype(np.int32)
        ids[3, 2] = -1
        got = ds4.indexed_mixed_attention_prefill(q, raw, comp, ids, sinks, pos0=pos0, window=window, ratio=ratio,
                                                  raw_start=raw_start)
        newest = pos0 + T - 1
        for t in range(T):
            rows = _walk_token(raw.astype(np.float32), comp.astype(np.float32), ids[t].tolist(), pos0 + t, newest,
                               window, ratio, raw_start).astype(np.float64)
            qh = torch.from_numpy(q[t]).to(torch.float16).to(torch.float64)
            logits = torch.cat([qh @ torch.from_numpy(rows).T * 512 ** -0.5,
                                torch.from_numpy(sinks.astype(np.float64))[:, None]], dim=1)
            prob = torch.softmax(logits, dim=1)[:, :-1]
            want = (prob @ torch.from_numpy(rows)).numpy() if rows.shape[0] else np.zeros((H, 512))
            np.testing.assert_allclose(got[t], want, rtol=1e-12, atol=1e-12, err_msg=f"{pos0} {t}")
        if raw_start == 0 and ratio != 0:
            # ascending ids: the composed form's filter selects the rows the kernel's stop rule does; its
            # float16 sinks move the result by at most the rounding of the sink logit
            ref = ds4.indexed_mixed_attention_prefill_reference(q, raw, comp, ids, sinks, pos0=pos0, window=window,
                                                                ratio=ratio)
            np.testing.assert_allclose(ref, got, rtol=0, atol=2e-3)
    # unsorted ids: the kernel stops at the first invisible id, the composed form only drops it
    raw = (rng.standard_normal((8, 512)) * 0.5).astype(np.float16)
    ids = np.tile(np.array([[1, 29, 0]], np.int32), (8, 1))          # visible = (qpos+1)//4 <= 4 < 29
    stop = ds4.indexed_mixed_attention_prefill(q[:8], raw, comp, ids, sinks, pos0=8, window=128, ratio=4)
    filt = ds4.indexed_mixed_attention_prefill_reference(q[:8], raw, comp, ids, sinks, pos0=8, window=128, ratio=4)
    only_first = ds4.indexed_mixed_attention_prefill(q[:8], raw, comp, ids[:, :1], sinks, pos0=8, window=128, ratio=4)
    both = ds4.indexed_mixed_attention_prefill(q[:8], raw, comp, ids[:, [0, 2]], sinks, pos0=8, window=128, ratio=4)
    np.testing.assert_array_equal(stop, only_first)
    np.testing.assert_allclose(filt, both, rtol=0, atol=2e-3)
    assert np.abs(filt - stop).max() > 1e-2


def test_fused_decode_prep_all_tie_integer_and_row_parts():
    # reference tests/test_deepseek_v4_decode_attention_kernel.py:215-243: equal scores select arange(topk)
    inv = ds4.rope_inverse_frequencies(64, ds4.DS4_COMPRESS_ROPE_BASE, ds4.DS4_YARN).astype(np.float32)
    H, N, K = 8, 50, 7
    q = np.zeros((H, 128), np.float32)
    pooled = np.ones((N, 128), np.float32)
    w = np.ones(H, np.float32)
    kv = np.zeros(512, np.float16)
    params = np.array([100, 0], np.int32)
    sel, row, scores = ds4.fused_decode_prep(q, pooled, w, kv, inv, params, scale=128 ** -0.5, topk=K)
    np.testing.assert_array_equal(sel, np.arange(K))
    assert np.all(scores == 0) and np.all(row == 0)
    # q = ones: the QAT row is [12, 0, ...] exactly (Hadamard of ones), so score(r) = sum_h w_h relu(12 p_r0) scale
    # computable by hand; distinct integers in column 0 give a known order, equal ones tie to the lower row
    q = np.ones((H, 128), np.float32)
    rng = np.random.default_rng(3)
    col0 = rng.integers(-3, 6, N).astype(np.float32)
    pooled = np.zeros((N, 128), np.float32)
    pooled[:, 0] = col0
    pooled[:, 1:] = rng.integers(-2, 3, (N, 127))                 # multiplied by exact zeros of the QAT row
    w = (rng.integers(1, 5, H) * 0.25).astype(np.float32)
    sel, _, scores = ds4.fused_decode_prep(q, pooled, w, kv, inv, params, scale=0.5, topk=K)
    by_hand = np.maximum(12.0 * col0.astype(np.float64), 0.0) * 0.5 * w.astype(np.float64).sum()
    np.testing.assert_allclose(scores, by_hand, rtol=0, atol=1e-9)
    order = np.lexsort((np.arange(N), -by_hand))[:K]
    thr = by_hand[order[-1]]
    above = np.nonzero(by_hand > thr)[0]
    ties = np.nonzero(by_hand == thr)[0][:K - above.size]
    np.testing.assert_array_equal(sel, np.concatenate([above, ties]))   # emission: above ascending, then ties
    # prepared row = FP8 round trip of the first 448 columns + rope of the last 64 at float16 rounding
    kv = (rng.standard_normal(512) * 0.3).astype(np.float16)
    _, row, _ = ds4.fused_decode_prep(q, pooled, w, kv, inv, np.array([3844, 0], np.int32), scale=0.5, topk=K)
    head = ds4.fp8_kv_roundtrip(kv.astype(np.float32))[:448].astype(np.float16)
    np.testing.assert_array_equal(row[:448].view(np.uint16), head.view(np.uint16))
    # (float16 rounding of cos/sin, of the four products and of the two sums: within 2e-3 of the float64 rotation)
    x = kv[448:].astype(np.float64).reshape(32, 2)
    ang = 3844.0 * inv.astype(np.float64)
    want = np.stack([x[:, 0] * np.cos(ang) - x[:, 1] * np.sin(ang), x[:, 0] * np.sin(ang) + x[:, 1] * np.cos(ang)], 1)
    np.testing.assert_allclose(row[448:].astype(np.float64), want.reshape(-1), rtol=0, atol=2e-3)
    assert np.abs(row[448:].astype(np.float64) - kv[448:].astype(np.float64)).max() > 0.05    # it did rotate


def test_torch_restatement_of_the_decode_layer_matches_the_numpy_oracle():
    """oracle/ds4_torch.py (the threaded CPU baseline that bench.py times) against the float64 NumPy oracle on a
    reduced layer: scores to float32 accuracy, the selected set exactly (including a block of tied scores, which
    go to the lower rows), the attention output to 1e-5."""
    import torch

    from oracle import ds4_torch

    rng = np.random.default_rng(12)
    H, N, TOPK, WIN, NT = 64, 2048, 128, 32, 8192
    qi = ds4.round_bf16(rng.standard_normal((1, H, 128), dtype=np.float32))
    k32 = rng.standard_normal((1, N, 128), dtype=np.float32)
    k32[0, 700:716] = k32[0, 700]                      # sixteen identical keys: tied scores
    ks = (np.abs(k32).max(-1) / 448).astype(np.float32)
    codes = ds4.e4m3_encode(k32 / ks[..., None])
    w = rng.uniform(0, 1, (1, H)).astype(np.float32)
    q = ds4.round_bf16(rng.standard_normal((1, H, 576), dtype=np.float32))
    kv = ds4.round_bf16(rng.standard_normal((1, NT, 576), dtype=np.float32))
    t = torch.from_numpy
    s64 = ds4.indexer_scores_fp8(qi, codes, ks, w)
    s32 = ds4_torch.indexer_scores_fp8(t(qi[0]), t(codes[0]), t(ks[0]), t(w[0])).numpy()
    np.testing.assert_allclose(s32, s64[0], rtol=1e-5, atol=1e-4)
    # selection on the same float32 scores: identical sets, ties to the lower rows
    scores = s64[0].astype(np.float32)
    scores[700:716] = np.sort(scores)[-TOPK + 4]        # the tie block straddles the k-th place
    want_sel = np.sort(ds4.radix_select_topk(scores, TOPK))
    got_sel = ds4_torch.topk_rows(t(scores), TOPK).numpy()
    np.testing.assert_array_equal(got_sel, want_sel)
    assert (np.diff(got_sel) > 0).all()
    tied = [r for r in got_sel if 700 <= r < 716]
    assert tied == list(range(700, 700 + len(tied))) and 0 < len(tied) < 16
    # the whole layer
    sel = ds4.radix_select_topk(s32, TOPK).astype(np.int64)
    rows = np.concatenate([np.arange(NT - WIN, NT), 4 * np.sort(sel) + 3])[None]
    want = ds4.sparse_mla_decode(q, kv, rows, scale=576 ** -0.5)
    got = ds4_torch.decode_layer(t(qi[0]), t(codes[0]), t(ks[0]), t(w[0]), t(q[0]), t(kv[0]), topk=TOPK, window=WIN,
                                 scale=576 ** -0.5).numpy()
    np.testing.assert_allclose(got, want[0], rtol=1e-5, atol=1e-5)
