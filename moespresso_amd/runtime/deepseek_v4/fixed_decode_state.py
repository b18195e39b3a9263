"""Fixed-capacity decode state of the DS4 compressed-attention layers.

Mirror of the part of the reference module ``src/moespresso/runtime/deepseek_v4/fixed_decode_state.py``
that the attention hot path touches: the per-token parameter helpers ``decode_step_params`` and
``pad_scores_to_capacity`` (:186-206), the capacity buffers of the derived caches with their append
(``aux_capacity_buffer`` :209, ``aux_fixed_update`` :215-288), and the branch object that carries them.
The reference keeps shapes fixed so that a compiled decode island is not retraced when the pool gains a
row; here the same layout keeps a captured HIP graph valid: pool rows live in buffers of
``ceil(max_context / ratio)`` rows, the number of rows in use travels in a small int32 array on the
device (``DecodeStepParams``), and the kernels read it there (``fused_decode_prep`` /
``fused_decode_sdpa`` with ``pool_rows_in_params=True``). The window-accumulator half of the reference
module (compressor state, :300-657) belongs to the model's compressor and is not part of this package.
"""

from __future__ import annotations

import math
import os

import torch

_FIXED_STATE_ENV = "MOESPRESSO_DSV4_DECODE_FIXED_STATE"
_MAX_CONTEXT_ENV = "MOESPRESSO_DSV4_DECODE_MAX_CONTEXT"
_DEFAULT_MAX_CONTEXT = 4096


def fixed_decode_state_enabled() -> bool:
    """Kill switch read per call: ``MOESPRESSO_DSV4_DECODE_FIXED_STATE=0`` keeps the growing layout (reference :90)."""
    return os.environ.get(_FIXED_STATE_ENV, "1") != "0"


def fixed_decode_max_context() -> int:
    """Maximum context that sizes the capacity buffers (reference :96)."""
    return int(os.environ.get(_MAX_CONTEXT_ENV, str(_DEFAULT_MAX_CONTEXT)))


class _FixedAux:
    """One derived cache (FP8-rounded or QAT'd pool rows) in a capacity buffer (reference :101)."""

    __slots__ = ("cap", "rows", "view")

    def __init__(self) -> None:
        self.cap = None
        self.rows = 0
        self.view = None


class _FixedBranchState:
    """Capacity and derived caches of one compressor state dict (the fields of reference :113 that the
    attention path reads)."""

    __slots__ = ("ratio", "pool_capacity", "aux", "engaged_pos")

    def __init__(self, *, ratio: int, pool_capacity: int | None = None, max_context: int | None = None) -> None:
        self.ratio = int(ratio)
        if pool_capacity is None:
            ctx = fixed_decode_max_context() if max_context is None else int(max_context)
            pool_capacity = int(math.ceil(ctx / self.ratio)) if self.ratio > 0 else 0
        self.pool_capacity = int(pool_capacity)
        self.aux: dict[str, _FixedAux] = {}
        self.engaged_pos: int | None = None


def aux_capacity_buffer(branch: _FixedBranchState, name: str):
    """Full capacity buffer of a derived cache, or None before its first update (reference :209)."""
    aux = branch.aux.get(name)
    return None if aux is None else aux.cap


def aux_fixed_update(branch: _FixedBranchState, state: dict, *, name: str, rows_key: str, pooled, transform):
    """Append ``transform(new pool rows)`` to a derived cache held in a capacity buffer (reference :215-288).

    ``pooled`` ``[B, rows, W]`` is the pool in use; rows already transformed are kept, only the tail goes
    through ``transform``. The legacy keys ``state[name]`` / ``state[rows_key]`` are republished as the
    in-use view, and adopted when they were set behind the buffer's back. Returns ``(view, prior_rows)``,
    or None when the fixed layout cannot serve (capacity exceeded, malformed legacy cache, element type
    changed): the caller then uses the growing layout, which trusts the legacy keys.
    """
    rows = int(pooled.shape[1])
    if rows > branch.pool_capacity:
        return None
    aux = branch.aux.get(name)
    cached_obj = state.get(name)
    cached_rows = int(state.get(rows_key, 0) or 0)
    if aux is None or cached_obj is not aux.view or cached_rows != aux.rows:
        aux = _FixedAux()
        if cached_obj is not None and cached_rows > 0:
            if cached_rows > branch.pool_capacity or cached_rows > rows or int(cached_obj.shape[1]) != cached_rows:
                return None
            aux.cap = torch.zeros((int(cached_obj.shape[0]), branch.pool_capacity, int(cached_obj.shape[-1])),
                                  dtype=cached_obj.dtype, device=cached_obj.device)
            aux.cap[:, :cached_rows] = cached_obj
            aux.rows = cached_rows
        branch.aux[name] = aux
    prior_rows = aux.rows
    if rows < aux.rows:  # the pool shrank without a trim reset: start over
        aux.rows = 0
        prior_rows = 0
    if rows > aux.rows:
        tail = transform(pooled[:, aux.rows:, :])
        if aux.cap is None:
            aux.cap = torch.zeros((int(tail.shape[0]), branch.pool_capacity, int(tail.shape[-1])),
                                  dtype=tail.dtype, device=tail.device)
        elif tail.dtype != aux.cap.dtype:
            branch.aux.pop(name, None)
            return None
        if int(tail.shape[1]):
            aux.cap[:, aux.rows:rows] = tail
        aux.rows = rows
    if aux.cap is None:
        aux.cap = torch.zeros((int(pooled.shape[0]), branch.pool_capacity, int(pooled.shape[-1])),
                              dtype=pooled.dtype, device=pooled.device)
    view = aux.cap[:, :rows]
    aux.view = view
    state[name] = view
    state[rows_key] = rows
    return view, prior_rows


class DecodeStepParams:
    """The per-token scalars of the fused decode island as data on the device: int32 ``[position, ring write
    index, pool rows in use]`` in one persistent tensor, so that kernels recorded into a HIP graph read
    this token's values at replay. ``set`` copies from pinned host memory on the current stream (a copy
    node outside the captured region; nothing here allocates per token)."""

    def __init__(self, device):
        self.tensor = torch.zeros((3,), dtype=torch.int32, device=device)
        self._host = torch.zeros((3,), dtype=torch.int32, pin_memory=torch.device(device).type == "cuda")

    def set(self, *, offset: int, write_idx: int, pool_rows: int) -> torch.Tensor:
        self._host[0], self._host[1], self._host[2] = int(offset), int(write_idx), int(pool_rows)
        self.tensor.copy_(self._host, non_blocking=False)
        return self.tensor


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
