"""Per-token parameter helpers of the DS4 fixed-capacity decode state.

Mirror of ``decode_step_params`` and ``pad_scores_to_capacity`` of the reference module
``src/moespresso/runtime/deepseek_v4/fixed_decode_state.py`` (:186-206): the only two functions of
that module the attention hot path calls. The branch/adoption bookkeeping of the reference module is
cache management and is not part of this package.
"""

from __future__ import annotations

import torch


def decode_step_params(_xp=None, *, offset: int, pool_rows: int, device=None):
    """int32 ``[offset, pool_rows]`` on the device: position and valid-row count of one decode token,
    carried as data so that a captured graph reads them instead of baking them in (reference :186).

    The reference call sites pass their array-library module first (``decode_step_params(mx, offset=…,
    pool_rows=…)``); that positional is accepted and ignored."""
    return torch.tensor([int(offset), int(pool_rows)], dtype=torch.int32, device=device)


def pad_scores_to_capacity(*args):
    """Mask score columns at and past the valid-row count ``params[1]`` to ``-inf`` (reference :198):
    ``pad_scores_to_capacity(scores, params)``, or with the reference's leading array-module handle,
    ``pad_scores_to_capacity(mx, scores, params)``.

    Valid columns pass through bitwise. (``fused_score_tail`` applies the same mask in-kernel; this is
    the stand-alone form for score rows that come from another producer.)
    """
    if len(args) == 3 and not isinstance(args[0], torch.Tensor):
        args = args[1:]
    if len(args) != 2:
        raise TypeError("pad_scores_to_capacity takes (scores, params), optionally behind an array-module handle")
    scores, params = args
    if params.dtype != torch.int32 or params.numel() < 2:
        raise ValueError("params must be int32 [offset, pool_rows]")
    capacity = int(scores.shape[-1])
    valid = (torch.arange(capacity, dtype=torch.int32, device=scores.device) < params[1]).reshape(
        (1,) * (scores.ndim - 1) + (capacity,))
    return torch.where(valid, scores, torch.full((), float("-inf"), dtype=scores.dtype, device=scores.device))
