"""CPU mirror of the index arithmetic that turns a prefill token into row addresses (no GPU).

`sparse_attn_prefill_kernel` and the per-token form of `sparse_attn_split_kernel` build, for every token, a table of
row pointers: ring rows `(raw_start + win_first + slot) wrapped once at raw_cap`, pool rows `id * row_mul + row_add`
for ids that pass the range check, a zero row otherwise. A pointer outside its tensor is a memory fault on the
GPU, so the arithmetic (the unsigned 32-bit window rules of the reference kernel,
indexed_attention_kernel.py:120-141, as `unit_of` in moespresso_amd/csrc/sparse_attn.hip restates them) is
replayed here in NumPy over random and extreme shapes, and every row index it yields is checked against the bounds
of the tensor it addresses, together with the sizes that the kernel's LDS tables assume.
"""

import numpy as np

U32 = np.uint32
K_TILE, K_MAX_TILES, K_MIN_TILES = 32, 22, 5


def unit_rows(t, *, pos0, n_tokens, raw_cap, raw_start, window, ratio, n_pool, host_n_win):
    """(ring row indices in slot order, visible pool prefix) of token t, in the kernel's arithmetic."""
    with np.errstate(over="ignore"):
        qpos = U32(pos0) + U32(t)
        n_raw = U32(raw_cap)
        last_pos = U32(pos0) + U32(n_tokens) - U32(1)
        first_raw_pos = last_pos + U32(1) - n_raw
        window_first = qpos + U32(1) - U32(window) if (window != 0 and qpos + U32(1) > U32(window)) else U32(0)
        first = max(first_raw_pos, window_first)
        last = min(qpos, last_pos)
        n_win = int(last - first + U32(1)) if first <= last else 0
        n_win = min(n_win, host_n_win)
        win_first = int(first - first_raw_pos) if first <= last else 0
    rows = []
    for ls in range(n_win):
        r = int(U32(raw_start) + U32(win_first) + U32(ls))
        if r >= raw_cap:
            r -= raw_cap
        rows.append(r)
    vis = n_pool if ratio == 0 else int((int(qpos) + 1) // ratio)
    return rows, min(vis, n_pool), n_win


def host_n_win(pos0, n_tokens, raw_cap, window):
    """Slot space the host sizes for the window part (mspr_indexed_mixed_attention_prefill)."""
    max_win = window if (window != 0 and window < raw_cap) else raw_cap
    return min(max_win, pos0 + n_tokens)


def check_shape(pos0, n_tokens, raw_cap, raw_start, window, ratio, n_pool, top_k, tokens):
    hw = host_n_win(pos0, n_tokens, raw_cap, window)
    fits = (hw + K_TILE - 1) // K_TILE + (top_k + K_TILE - 1) // K_TILE <= K_MAX_TILES
    for t in tokens:
        rows, vis, n_win = unit_rows(t, pos0=pos0, n_tokens=n_tokens, raw_cap=raw_cap, raw_start=raw_start,
                                     window=window, ratio=ratio, n_pool=n_pool, host_n_win=hw)
        assert all(0 <= r < raw_cap for r in rows), (t, rows[:4])
        assert len(set(rows)) == len(rows)                      # a token never visits a ring row twice
        assert 0 <= vis <= n_pool
        # the window is what the reference's rule says: positions [max(first_raw, qpos+1-window), min(qpos, last)]
        qpos, last_pos = pos0 + t, pos0 + n_tokens - 1
        first_raw = last_pos + 1 - raw_cap
        if first_raw >= 0:
            lo = max(first_raw, qpos + 1 - window if window else 0, 0)
            want = [(raw_start + p - first_raw) % raw_cap for p in range(lo, min(qpos, last_pos) + 1)]
            assert rows == want[:hw], (t, rows[:4], want[:4])
        else:
            assert rows == []                                   # a ring deeper than the positions seen: nothing
        if fits:
            wt = (n_win + K_TILE - 1) // K_TILE
            for stop in (0, top_k // 2, top_k):
                n_tiles = max(K_MIN_TILES, wt + (stop + K_TILE - 1) // K_TILE)
                assert n_tiles <= K_MAX_TILES and n_tiles * K_TILE <= K_MAX_TILES * K_TILE
                # the first three tiles of a unit are requested from the unit before it: they exist
                assert n_tiles >= 3


def test_anchor_and_test_shapes():
    for shape in (
        dict(pos0=5000, n_tokens=3844, raw_cap=3900, raw_start=1234, window=128, ratio=4, n_pool=2300, top_k=512),
        dict(pos0=5000, n_tokens=3844, raw_cap=3844, raw_start=0, window=128, ratio=128, n_pool=69, top_k=69),
        dict(pos0=0, n_tokens=3844, raw_cap=3844, raw_start=0, window=128, ratio=4, n_pool=961, top_k=512),
        dict(pos0=28000, n_tokens=3844, raw_cap=3844, raw_start=0, window=128, ratio=4, n_pool=7961, top_k=512),
        dict(pos0=4000, n_tokens=300, raw_cap=340, raw_start=123, window=128, ratio=4, n_pool=900, top_k=256),
        dict(pos0=9000, n_tokens=700, raw_cap=760, raw_start=31, window=128, ratio=4, n_pool=2000, top_k=512),
        dict(pos0=100, n_tokens=40, raw_cap=72, raw_start=50, window=16, ratio=4, n_pool=64, top_k=24),
        dict(pos0=7000, n_tokens=300, raw_cap=900, raw_start=77, window=600, ratio=4, n_pool=1500, top_k=512),
    ):
        check_shape(**shape, tokens=range(shape["n_tokens"]))


def test_random_and_extreme_shapes():
    rng = np.random.default_rng(3)
    for _ in range(400):
        n_tokens = int(rng.integers(1, 300))
        raw_cap = int(rng.integers(1, 400))
        pos0 = int(rng.choice([0, 1, int(rng.integers(0, 5000)), 2 ** 31 - 1 - n_tokens]))
        window = int(rng.choice([0, 1, 16, 128, int(rng.integers(1, 700))]))
        ratio = int(rng.choice([0, 1, 4, 128]))
        n_pool = int(rng.integers(1, 3000))
        check_shape(pos0, n_tokens, raw_cap, int(rng.integers(0, raw_cap)), window, ratio, n_pool,
                    int(rng.integers(0, 600)), tokens=range(0, n_tokens, max(1, n_tokens // 7)))
