"""GPU parity under large logits: the rescale branch of the lazily advanced softmax maximum.

Every attention kernel here keeps a reference maximum per query that moves only when a 32-key tile exceeds it by
more than a threshold in log2 units (8 where the softmax weights are float16, 64 where they are bfloat16), and then
rescales the denominator and the output accumulator. With N(0,1) data the logits have a spread of about one log2
unit, so after a query's first tile the branch never runs. Two kinds of data make it run with a non-empty
accumulator:

* a ramp: keys are `s_i * u + noise` along the visit order with `s_i` growing linearly, queries are
  `a_h * A * u + noise` with `a_h` in [1, 2], so the logit of every head grows by more than the threshold from
  each 32-key tile to the next (`ramp_step` below is the growth per tile of the slowest head): every tile after a
  query's first one takes the branch, however the keys are split into ranges;
* random data with queries scaled up (logit spread of 8-9 log2 units): the branch runs on some tiles and not on
  others, and in some waves of a workgroup and not in others.

Outputs are compared with the float64 oracle: 2e-3 absolute, the bar of the ordinary parity tests, plus a term for
the 16-bit roundings that the kernels are allowed (softmax weights, per-range partials, the output itself: each at
most eps = 2^-11 of the value it rounds in float16 (11 significant bits), 2^-8 in bfloat16 (8 bits)). With a softmax that a few keys dominate
these roundings do not average out as they do over thousands of comparable keys, and ramp data gives values of
magnitude up to a hundred, so the term is relative: a rounding of the weights or of a value moves an output by at
most eps * A, where A = sum_i p_i |v_i| is the attention over the absolute values (the float64 oracle run on |V|;
A >= |output|). `_close` allows three such roundings. The prefill consumer writes float32 and is held to the
reference's own rtol = atol = 2e-3, the 8-bit prefix form to its 1e-2.
"""

import numpy as np
import pytest
import torch

from oracle import ds4, qwen

pytestmark = pytest.mark.gpu

LOG2E = 1.4426950408889634


def _dev():
    return torch.device("cuda:0")


def _t(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(_dev())


def _close(got, want, dtype, abs_attention):
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    err = np.abs(got - want)
    bound = 2e-3 + 3.0 * eps * abs_attention
    assert (abs_attention >= np.abs(want) - 1e-9).all()
    assert (err <= bound).all(), (err.max(), np.abs(want).max(), (err / bound).max())


def _mla_abs_attention(q, kv, rows, scale):
    """sum_i p_i |v_i| of the gathered decode attention (weights of the float64 softmax, V = first 512 columns)."""
    out = np.empty((q.shape[0], q.shape[1], 512))
    for b in range(q.shape[0]):
        k = kv[b][rows[b]].astype(np.float64)
        logits = (q[b].astype(np.float64) @ k.T) * scale
        p = np.exp(logits - logits.max(axis=1, keepdims=True))
        out[b] = (p / p.sum(axis=1, keepdims=True)) @ np.abs(k[:, :512])
    return out


def _ramp(rng, n_queries, n_keys, dim, *, scale, ramp_step, amp=4.0, noise=0.1):
    """Queries [n_queries, dim] and keys [n_keys, dim] (float32) whose logits `scale * q.k` grow along the key
    index by at least `ramp_step` log2 units per 32 keys for every query."""
    u = rng.standard_normal(dim)
    u /= np.linalg.norm(u)
    a = rng.uniform(1.0, 2.0, size=(n_queries, 1))
    q = a * amp * u[None, :] + noise * rng.standard_normal((n_queries, dim))
    # slowest query: a = 1, and the noise of q projects on the key direction with a spread of `noise`
    slope = 1.25 * ramp_step / (32.0 * LOG2E * scale * (amp - 3.0 * noise))
    s = slope * np.arange(n_keys, dtype=np.float64)
    k = s[:, None] * u[None, :] + noise * rng.standard_normal((n_keys, dim))
    return q.astype(np.float32), k.astype(np.float32)


def _min_tile_growth(q, k, scale):
    """Smallest growth (log2 units) of the per-tile maximum logit from one 32-key tile to the next, over queries."""
    logits = (q.astype(np.float64) @ k.astype(np.float64).T) * scale * LOG2E
    n = (logits.shape[1] // 32) * 32
    tile_max = logits[:, :n].reshape(logits.shape[0], -1, 32).max(axis=2)
    return np.diff(tile_max, axis=1).min()


# ------------------------------------------------------------------ sparse MLA decode (split kernel + merge)

@pytest.mark.parametrize("dtype,k_dim,batch,ramp_step", [
    (torch.float16, 512, 64, 8.5),     # four key ranges per sequence: window tile + two gathered tiles each
    (torch.float16, 576, 64, 8.5),
    (torch.bfloat16, 576, 64, 65.0),
    (torch.bfloat16, 512, 64, 65.0),
    (torch.float16, 512, 256, 8.5),    # one key range per sequence: the split kernel normalises and stores
    (torch.bfloat16, 576, 256, 65.0),
])
def test_sparse_mla_decode_ramp(dtype, k_dim, batch, ramp_step):
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    n_pool, n_rows, win_rows, heads = 400, 256, 64, 64
    rng = np.random.default_rng(17 + k_dim + batch)
    scale = k_dim ** -0.5
    q = np.empty((batch, heads, k_dim), np.float32)
    kv = np.empty((batch, n_pool, k_dim), np.float32)
    rows = np.empty((batch, n_rows), np.int32)
    for b in range(batch):
        q[b], kv[b] = _ramp(rng, heads, n_pool, k_dim, scale=scale, ramp_step=ramp_step,
                            amp=8.0 if dtype == torch.bfloat16 else 4.0)
        rows[b] = np.sort(rng.choice(np.arange(win_rows, n_pool), size=n_rows, replace=False))
    qt, kvt = _t(q, dtype), _t(kv, dtype)
    qr, kvr = qt.float().cpu().numpy(), kvt.float().cpu().numpy()
    # the data does what it is for: visited keys in visit order (window rows, then the gathered ones)
    order = np.concatenate([np.arange(win_rows), rows[0]])
    assert _min_tile_growth(qr[0], kvr[0][order], scale) > (64.0 if dtype == torch.bfloat16 else 8.0)
    got = iak.sparse_mla_decode(qt, kvt, _t(rows), scale=scale, window_start=0, window_rows=win_rows)
    all_rows = np.concatenate([np.tile(np.arange(win_rows, dtype=np.int32), (batch, 1)), rows], axis=1)
    want = ds4.sparse_mla_decode(qr, kvr, all_rows, scale=scale)
    got = got.float().cpu().numpy()
    assert np.isfinite(got).all()
    _close(got, want, dtype, _mla_abs_attention(qr, kvr, all_rows, scale))


@pytest.mark.parametrize("dtype,q_scale", [(torch.float16, 6.0), (torch.bfloat16, 48.0)])
def test_sparse_mla_decode_scaled_random_queries(dtype, q_scale):
    """Random rows, queries scaled so that the logit spread is of the order of the threshold: some tiles move the
    maximum, most do not."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    batch, heads, k_dim, n_pool, n_rows, win_rows = 16, 64, 576, 3000, 2048, 128
    rng = np.random.default_rng(5)
    q = (q_scale * rng.standard_normal((batch, heads, k_dim))).astype(np.float32)
    kv = rng.standard_normal((batch, n_pool, k_dim)).astype(np.float32)
    rows = np.stack([rng.choice(n_pool, size=n_rows, replace=False) for _ in range(batch)]).astype(np.int32)
    qt, kvt = _t(q, dtype), _t(kv, dtype)
    scale = k_dim ** -0.5
    got = iak.sparse_mla_decode(qt, kvt, _t(rows), scale=scale, window_start=n_pool - win_rows, window_rows=win_rows)
    win = np.tile(np.arange(n_pool - win_rows, n_pool, dtype=np.int32), (batch, 1))
    qr, kvr, all_rows = qt.float().cpu().numpy(), kvt.float().cpu().numpy(), np.concatenate([win, rows], axis=1)
    want = ds4.sparse_mla_decode(qr, kvr, all_rows, scale=scale)
    got = got.float().cpu().numpy()
    assert np.isfinite(got).all()
    _close(got, want, dtype, _mla_abs_attention(qr, kvr, all_rows, scale))


# ------------------------------------------------------------------ DS4 prefill consumer (persistent kernel)

def _prefill_ramp_case(rng, tokens, raw_cap, n_comp, heads, raw_start, ramp_step):
    """Ring rows ramp with their position, pool rows continue the ramp above the newest ring row; ascending ids."""
    scale = 512 ** -0.5
    q2, rows = _ramp(rng, tokens * heads, raw_cap + n_comp, 512, scale=scale, ramp_step=ramp_step)
    q = np.ascontiguousarray(q2.reshape(tokens, heads, 512).transpose(1, 0, 2))[None]  # [1, H, T, 512]
    raw = np.empty((1, 1, raw_cap, 512), np.float32)
    raw[0, 0, (raw_start + np.arange(raw_cap)) % raw_cap] = rows[:raw_cap]  # logical row i at (raw_start + i) % cap
    comp = rows[raw_cap:][None]
    return q, raw.astype(np.float16), comp.astype(np.float16)


@pytest.mark.parametrize("q_dtype", [torch.float16, torch.float32])
def test_prefill_consumer_ramp(q_dtype):
    """Every tile of every token exceeds the common maximum by more than 2^8: the waves exchange their block
    maxima, rescale the denominators and the accumulator, and write P^T again on each of them."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    T, raw_cap, P, H, pos0, raw_start = 300, 340, 900, 64, 4000, 123
    rng = np.random.default_rng(41)
    q, raw, comp = _prefill_ramp_case(rng, T, raw_cap, P, H, raw_start, ramp_step=8.5)
    ids = np.stack([np.sort(rng.choice(P, size=256, replace=False)) for _ in range(T)])[None].astype(np.int32)
    sinks = rng.standard_normal((H,)).astype(np.float32)
    qt = _t(q, q_dtype)
    fn = iak.indexed_mixed_attention_prefill_live_f16 if q_dtype == torch.float16 else \
        iak.indexed_mixed_attention_prefill_live_f32
    kw = dict(pos0=pos0, window=128, ratio=4, raw_start=raw_start)
    got = fn(qt, _t(raw), _t(comp), _t(ids), _t(sinks), **kw).cpu().numpy()
    assert np.isfinite(got).all()
    qr = qt.float().cpu().numpy()
    for t in (0, 1, 2, 77, 150, 255, 256, 298, 299):
        raw_rows, comp_rows = ds4.indexed_visit_rows(raw_cap=raw_cap, n_comp=P, topk=ids[0, t], qpos=pos0 + t,
                                                     last_pos=pos0 + T - 1, window=128, ratio=4, raw_start=raw_start)
        rows = np.concatenate([raw[0, 0, raw_rows].astype(np.float32).reshape(-1, 512),
                               comp[0, comp_rows].astype(np.float32).reshape(-1, 512)], axis=0)
        assert len(raw_rows) == min(128, raw_cap - T + 1 + t) and len(comp_rows) == 256
        assert _min_tile_growth(ds4.round_f16(qr[0, :, t]), rows, 512 ** -0.5) > 8.0
        want = ds4.attend_rows_f64(ds4.round_f16(qr[0, :, t]), rows, sinks, 512 ** -0.5)
        np.testing.assert_allclose(got[0, :, t], want, rtol=2e-3, atol=2e-3, err_msg=f"token {t}")


def test_prefill_consumer_scaled_random_queries():
    """Random rows, queries scaled by 6: tiles that move the maximum and tiles that do not, blocks of a tile that
    raise the flag while the other blocks of the same tile do not."""
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    T, raw_cap, P, H, pos0, raw_start = 700, 760, 2000, 64, 9000, 31
    rng = np.random.default_rng(43)
    q = (6.0 * rng.standard_normal((1, H, T, 512))).astype(np.float16)
    raw = rng.standard_normal((1, 1, raw_cap, 512)).astype(np.float16)
    comp = rng.standard_normal((1, P, 512)).astype(np.float16)
    ids = np.stack([np.sort(rng.choice(P, size=512, replace=False)) for _ in range(T)])[None].astype(np.int32)
    sinks = rng.standard_normal((H,)).astype(np.float32)
    kw = dict(pos0=pos0, window=128, ratio=4, raw_start=raw_start)
    got = iak.indexed_mixed_attention_prefill_live_f16(_t(q), _t(raw), _t(comp), _t(ids), _t(sinks), **kw).cpu().numpy()
    assert np.isfinite(got).all()
    for t in (0, 1, 255, 256, 257, 511, 512, 698, 699):
        raw_rows, comp_rows = ds4.indexed_visit_rows(raw_cap=raw_cap, n_comp=P, topk=ids[0, t], qpos=pos0 + t,
                                                     last_pos=pos0 + T - 1, window=128, ratio=4, raw_start=raw_start)
        rows = np.concatenate([raw[0, 0, raw_rows].astype(np.float32).reshape(-1, 512),
                               comp[0, comp_rows].astype(np.float32).reshape(-1, 512)], axis=0)
        want = ds4.attend_rows_f64(q[0, :, t].astype(np.float32), rows, sinks, 512 ** -0.5)
        np.testing.assert_allclose(got[0, :, t], want, rtol=2e-3, atol=2e-3, err_msg=f"token {t}")


# ------------------------------------------------------------------ Qwen flash prefill (dense and Q8 prefix)

def _flash_ramp_case(rng, Hq, Hkv, L, past, ramp_step, amp):
    scale = 256 ** -0.5
    n = past + L
    q = np.empty((1, Hq, L, 256), np.float32)
    k = np.empty((1, Hkv, n, 256), np.float32)
    v = (0.5 * rng.standard_normal((1, Hkv, n, 256))).astype(np.float32)
    rep = Hq // Hkv
    for kvh in range(Hkv):
        qq, kk = _ramp(rng, rep * L, n, 256, scale=scale, ramp_step=ramp_step, amp=amp)
        q[0, kvh * rep:(kvh + 1) * rep] = qq.reshape(rep, L, 256)
        k[0, kvh] = kk
    return q, k, v, scale


@pytest.mark.parametrize("dtype,L,past,ramp_step", [
    (torch.bfloat16, 96, 160, 65.0),
    (torch.float16, 96, 160, 8.5),
    (torch.bfloat16, 64, 1200, 65.0),    # short chunk over a deep prefix: key-range splits + merge
    (torch.float16, 64, 1200, 8.5),
    (torch.bfloat16, 300, 0, 65.0),      # no prefix: the diagonal tiles are the only ones
])
def test_flash_prefill_ramp(dtype, L, past, ramp_step):
    from moespresso_amd.runtime.qwen import kquant

    rng = np.random.default_rng(L + past)
    q, k, v, scale = _flash_ramp_case(rng, 16, 2, L, past, ramp_step, amp=8.0 if dtype == torch.bfloat16 else 4.0)
    qt, kt, vt = _t(q, dtype), _t(k, dtype), _t(v, dtype)
    qr, kr, vr = qt.float().cpu().numpy(), kt.float().cpu().numpy(), vt.float().cpu().numpy()
    assert _min_tile_growth(qr[0, 0], kr[0, 0], scale) > (64.0 if dtype == torch.bfloat16 else 8.0)
    got = kquant.flash_prefill(qt, kt, vt, scale, past_len=past).float().cpu().numpy()
    assert np.isfinite(got).all()
    want = qwen.causal_prefill_attention(qr, kr, vr, scale, past=past)
    _close(got, want, dtype, qwen.causal_prefill_attention(qr, kr, np.abs(vr), scale, past=past))


@pytest.mark.parametrize("dtype,q_scale", [(torch.bfloat16, 30.0), (torch.float16, 5.0)])
def test_flash_prefill_scaled_random_queries(dtype, q_scale):
    from moespresso_amd.runtime.qwen import kquant

    L, past = 200, 700
    g = torch.Generator().manual_seed(77)
    q = (q_scale * torch.randn((1, 16, L, 256), generator=g)).to(dtype)
    k = torch.randn((1, 2, past + L, 256), generator=g).to(dtype)
    v = (0.5 * torch.randn((1, 2, past + L, 256), generator=g)).to(dtype)
    scale = 256 ** -0.5
    got = kquant.flash_prefill(q.to(_dev()), k.to(_dev()), v.to(_dev()), scale, past_len=past).float().cpu().numpy()
    assert np.isfinite(got).all()
    want = qwen.causal_prefill_attention(q.float().numpy(), k.float().numpy(), v.float().numpy(), scale, past=past)
    _close(got, want, dtype, qwen.causal_prefill_attention(q.float().numpy(), k.float().numpy(), v.float().abs().numpy(),
                                                           scale, past=past))


@pytest.mark.parametrize("past,L", [(300, 70), (700, 1100), (1100, 40)])
def test_sdpa_fa_prefill_q8_ramp(past, L):
    """The quantised-prefix form (short chunk: prefix unpacked in the kernel; long chunk: converted first; deep
    prefix under a short chunk: key-range splits), logits growing by more than 2^8 per tile. The oracle attends
    the dequantised prefix and the chunk rows as the kernel is given them; 1e-2 is the 8-bit KV bar."""
    from moespresso_amd.runtime.qwen import kquant

    rng = np.random.default_rng(past + L)
    q, k, v, scale = _flash_ramp_case(rng, 16, 2, L, past, 8.5, amp=4.0)
    dev = _dev()

    def words(w):
        return torch.from_numpy(np.ascontiguousarray(w).view(np.int32)).to(dev).view(torch.uint32)

    kq, ks, kb = qwen.affine_q8_quantize(k[:, :, :past])
    vq, vs, vb = qwen.affine_q8_quantize(v[:, :, :past])
    k_all = np.concatenate([qwen.affine_q8_dequantize(kq, ks, kb), k[:, :, past:]], axis=2)
    v_all = np.concatenate([qwen.affine_q8_dequantize(vq, vs, vb), v[:, :, past:]], axis=2)
    got = kquant.sdpa_fa_prefill_q8(_t(q), words(kq), _t(ks), _t(kb), words(vq), _t(vs), _t(vb), _t(k[:, :, past:]),
                                    _t(v[:, :, past:]), scale, bq=32, bk=16, stage=2).cpu().numpy()
    assert np.isfinite(got).all()
    assert _min_tile_growth(q[0, 0], k_all[0, 0], scale) > 8.0
    # the kernel stages the queries and the chunk's own rows in 16 bits: float16 next to a prefix that it unpacks
    # itself, bfloat16 (prefix included) for chunks of 1024 queries and more, whose prefix is converted beforehand
    stage = ds4.round_bf16 if L >= 1024 else ds4.round_f16
    if L >= 1024:
        k_all, v_all = stage(k_all), stage(v_all)
    want = qwen.causal_prefill_attention(stage(q), np.concatenate(
        [k_all[:, :, :past], stage(k_all[:, :, past:])], axis=2), np.concatenate(
        [v_all[:, :, :past], stage(v_all[:, :, past:])], axis=2), scale, past=past)
    err = np.abs(got - want).max()
    assert err < 1e-2, err
