"""Threaded CPU restatement of the sparse decode attention layer in torch (float32), for the CPU-baseline leg of
the benchmark.

TEST INFRASTRUCTURE ONLY, like the rest of this package: the benchmark's `cpu_baseline` times it on the host's
cores and tests/test_oracle_ds4.py pins it against the NumPy oracle (`oracle.ds4`: `indexer_scores_fp8`,
`radix_select_topk`, `sparse_mla_decode`). It states the same three steps as BASELINE configs 4 and 5 chained

    score[r] = sum_h w[h] * relu(q_idx[h] . e4m3(codes[r])) * key_scale[r]        (lightning indexer, fp8 keys)
    sel      = the top-k rows by score, ties to the lower row, in ascending row order
    out[h]   = softmax(q[h] . kv[rows] * scale) . kv[rows, :512]                  (window rows, then 4 sel + 3)

as dense tensor operations, so that the matrix products run on torch's threaded CPU kernels; `torch.set_num_threads`
decides how many cores it uses. The NumPy oracle computes in float64 and is the checker; this one is float32 and is
a baseline to be timed, not a reference for parity.
"""

from __future__ import annotations

import torch


def indexer_scores_fp8(q_idx: torch.Tensor, key_codes: torch.Tensor, key_scales: torch.Tensor,
                       weights: torch.Tensor) -> torch.Tensor:
    """q_idx f32 ``[H,128]`` (bf16 values), key_codes uint8 ``[N,128]`` (E4M3FN bytes), key_scales f32 ``[N]``,
    weights f32 ``[H]`` -> scores f32 ``[N]``."""
    keys = key_codes.view(torch.float8_e4m3fn).to(torch.float32)           # exact: every E4M3 value is a float32
    raw = q_idx @ keys.T                                                   # [H, N]
    return (torch.relu(raw) * weights[:, None]).sum(dim=0) * key_scales


def topk_rows(scores: torch.Tensor, k: int) -> torch.Tensor:
    """The k rows with the largest scores, ties to the lower row, ascending (a stable descending sort keeps the
    lower row first among equal scores)."""
    order = torch.sort(scores, descending=True, stable=True).indices[:k]
    return torch.sort(order).values


def sparse_mla_decode(q: torch.Tensor, kv: torch.Tensor, rows: torch.Tensor, scale: float, v_dim: int = 512) -> torch.Tensor:
    """q f32 ``[H,Dk]``, kv ``[N,Dk]`` (any float dtype), rows int64 ``[R]`` -> f32 ``[H,v_dim]``."""
    gathered = kv.index_select(0, rows).to(torch.float32)
    p = torch.softmax((q @ gathered.T) * scale, dim=-1)
    return p @ gathered[:, :v_dim]


def decode_layer(q_idx, key_codes, key_scales, weights, q, kv, *, topk: int, window: int, scale: float) -> torch.Tensor:
    """One sequence of the layer: indexer scores -> top-k -> attention over the last `window` cache rows followed by
    rows 4 sel + 3 (a compressed entry covers four cache rows; its last one is attended)."""
    sel = topk_rows(indexer_scores_fp8(q_idx, key_codes, key_scales, weights), topk)
    n = kv.shape[0]
    rows = torch.cat([torch.arange(n - window, n, dtype=torch.int64), 4 * sel + 3])
    return sparse_mla_decode(q, kv, rows, scale)
