"""CPU model of the arithmetic of the persistent prefill consumer (sparse_attn_prefill_kernel), against the oracle.

The kernel departs from the textbook online softmax in three ways that this model restates in NumPy: (1) the
running maximum of a head is a reference value that only moves when a tile exceeds it by more than 2^8 (log2
domain), (2) the softmax weights are rounded to float16 before they multiply V while the denominator sums the
unrounded float32 weights, (3) tokens are padded with fully masked tiles. The model shows that this arithmetic
stays within the tolerance of the GPU tests (2e-3) of the float64 oracle; the GPU tests check the kernel itself.
"""
import numpy as np

from oracle import ds4

TILE = 32
K_GROW = 8.0


def _visited_rows(t, pos0, n_tokens, raw, raw_start, comp, ids, window, ratio):
    """Rows a token visits, in the kernel's slot order: ring rows of the window, then ids up to the stop rule."""
    raw_cap = raw.shape[0]
    qpos, last_pos = pos0 + t, pos0 + n_tokens - 1
    first_raw_pos = last_pos + 1 - raw_cap
    first = max(first_raw_pos, qpos + 1 - window, 0)
    rows = [raw[(raw_start + (p - first_raw_pos)) % raw_cap] for p in range(first, min(qpos, last_pos) + 1)]
    visible = min((qpos + 1) // ratio, comp.shape[0])
    gathered = []
    for i in ids[t]:
        if i < 0:
            gathered.append(None)  # a skipped slot still occupies its place in the tile
            continue
        if i >= visible:
            break
        gathered.append(comp[i])
    return rows, gathered


def _tiles(rows, gathered, min_tiles=5):
    """32-slot tiles: the window padded to whole tiles, then the gathered slots, then masked tiles up to min_tiles."""
    slots = list(rows) + [None] * (-len(rows) % TILE) + list(gathered)
    slots += [None] * (-len(slots) % TILE)
    while len(slots) < min_tiles * TILE:
        slots += [None] * TILE
    return [slots[i:i + TILE] for i in range(0, len(slots), TILE)]


def consumer_model(q, tiles, sinks):
    """q float16 [H, 512]; tiles of 32 slots (float16 rows or None); sinks float32 [H] -> float32 [H, 512]."""
    H = q.shape[0]
    scale_log2 = np.float32(1.4426950408889634 / np.sqrt(512.0))
    m = np.full(H, -np.inf, dtype=np.float32)
    l = np.zeros(H, dtype=np.float32)
    o = np.zeros((H, 512), dtype=np.float32)
    qf = q.astype(np.float32)
    for tile in tiles:
        valid = np.array([r is not None for r in tile])
        k = np.stack([r if r is not None else np.zeros(512, np.float16) for r in tile]).astype(np.float32)
        s = (qf @ k.T).astype(np.float32) * scale_log2                      # [H, 32], float32 accumulation
        s = np.where(valid[None, :], s, -np.inf).astype(np.float32)
        tmax = s.max(axis=1)
        grow = tmax > m + np.float32(K_GROW)                                 # (-inf + 8 = -inf: any finite value grows)
        if grow.any():
            m_new = np.where(grow, tmax, m)
            with np.errstate(invalid="ignore"):
                alpha = np.where(grow, np.exp2(m - m_new), np.float32(1.0)).astype(np.float32)
            alpha = np.where(np.isnan(alpha), np.float32(0.0), alpha)
            l *= alpha
            o *= alpha[:, None]
            m = m_new
        m_safe = np.where(np.isinf(m), np.float32(0.0), m)
        p = np.exp2(s - m_safe[:, None]).astype(np.float32)
        l += p.sum(axis=1, dtype=np.float32)
        o += p.astype(np.float16).astype(np.float32) @ k                      # weights rounded to the element type
    sink = sinks.astype(np.float32) * np.float32(1.4426950408889634)
    m_all = np.maximum(m, sink)
    m_safe = np.where(np.isinf(m_all), np.float32(0.0), m_all)
    w = np.exp2(m - m_safe)
    den = l * w + np.exp2(sink - m_safe)
    f = np.where(den == 0, np.float32(0.0), w / den)
    return (o * f[:, None]).astype(np.float32)


def _case(seed, tokens, n_comp, heads, topk, window, pos0, raw_cap, raw_start, scale=1.0):
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((heads, tokens, 512), dtype=np.float32) * scale).astype(np.float16)
    raw = rng.standard_normal((raw_cap, 512), dtype=np.float32).astype(np.float16)
    comp = rng.standard_normal((n_comp, 512), dtype=np.float32).astype(np.float16)
    ids = np.stack([np.sort(rng.choice(n_comp, size=topk, replace=False)) for _ in range(tokens)]).astype(np.int32)
    ids[1, 3] = -1  # a skipped slot
    sinks = rng.standard_normal((heads,), dtype=np.float32)
    return q, raw, comp, ids, sinks, dict(pos0=pos0, window=window, ratio=4, raw_start=raw_start)


def test_model_of_the_prefill_consumer_stays_within_the_gpu_tolerance():
    tokens = 10
    q, raw, comp, ids, sinks, kw = _case(3, tokens, 90, 16, 70, 48, 300, 64, 17)
    want = ds4.indexed_mixed_attention_prefill(q.transpose(1, 0, 2).astype(np.float32), raw, comp, ids, sinks, **kw)
    for t in range(tokens):
        rows, gathered = _visited_rows(t, kw["pos0"], tokens, raw, kw["raw_start"], comp, ids, kw["window"], kw["ratio"])
        got = consumer_model(q[:, t], _tiles(rows, gathered), sinks)
        np.testing.assert_allclose(got, want[t], rtol=2e-3, atol=2e-3, err_msg=f"token {t}")


def test_model_with_large_scores_takes_the_rescale_path_more_than_once():
    # queries scaled up: tile maxima differ by far more than 2^8 from tile to tile, so the reference maximum moves
    # several times per token and float16 weights of earlier tiles get rescaled
    tokens = 4
    q, raw, comp, ids, sinks, kw = _case(5, tokens, 200, 8, 150, 32, 1000, 40, 3, scale=6.0)
    want = ds4.indexed_mixed_attention_prefill(q.transpose(1, 0, 2).astype(np.float32), raw, comp, ids, sinks, **kw)
    for t in range(tokens):
        rows, gathered = _visited_rows(t, kw["pos0"], tokens, raw, kw["raw_start"], comp, ids, kw["window"], kw["ratio"])
        got = consumer_model(q[:, t], _tiles(rows, gathered), sinks)
        np.testing.assert_allclose(got, want[t], rtol=2e-3, atol=2e-3, err_msg=f"token {t}")


def test_model_of_a_token_without_rows_returns_zeros():
    got = consumer_model(np.ones((4, 512), np.float16), _tiles([], []), np.zeros(4, np.float32))
    assert got.shape == (4, 512) and not got.any()
