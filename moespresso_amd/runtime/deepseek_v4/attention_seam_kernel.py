"""Fused DS4 attention seam: the partial rotary embedding in one launch.

Mirror of the reference module
``src/moespresso/runtime/deepseek_v4/attention_seam_kernel.py``: the same environment gates
(:141-163), eligibility contract (:200-244) and ``fused_partial_rope`` signature (:247). Each
partial-rope call site of the decode and prefill paths (query rope, KV rope, inverse rope on the
attention output, indexer query rope, pooled-row rope) is one HIP launch that reproduces the
composed operation sequence rounding for rounding: float32 angle ``position * inv_freq[p]``,
float32 cosine/sine cast to the element type (the inverse form negates the float32 sine first),
every product and sum of the rotation rounded to the element type, the leading channels copied.

Two operand forms, as in the reference: the offset form stands for ``arange(offset, offset + L)``
(engaged only while ``offset + L`` stays inside float32's exact-integer range), the positions form
takes the caller's float32 positions row.
"""

from __future__ import annotations

import os

import torch

from moespresso_amd import _lib

_FAMILY_ENV_FLAG = "MOESPRESSO_DSV4_ATTN_SEAM_FUSED"
_ROPE_ENV_FLAG = "MOESPRESSO_DSV4_ATTN_SEAM_ROPE"
_PREFILL_ENV_FLAG = "MOESPRESSO_DSV4_SEAM_ROPE_PREFILL"

_ROPE_DIM = 64
_ROPE_FREQS = _ROPE_DIM // 2

# Decode row cap (64 query heads is the widest served decode call); it is the eligibility contract
# when the prefill extension is switched off (reference :62-65).
_MAX_ROWS_DECODE = 64
# Structural ceiling for prefill-shaped calls: rows are counted in 32-bit, offsets in 64-bit (:67-73).
_MAX_ROWS_PREFILL = (1 << 31) - 1
# The offset form reproduces a float32 arange, exact only below 2**24 (:75-78).
_MAX_EXACT_POSITION = 1 << 24

# Operand forms that have been launched, keyed like the reference's pipeline cache (form, inverse).
_ROPE_KERNELS: dict[tuple[str, bool], str] = {}


def _metal_available() -> bool:
    """Name kept from the reference; reports whether the HIP device and kernel library are usable."""
    return _lib.hip_available()


def rope_seam_enabled() -> bool:
    """True when the fused rope seam may engage (reference :141)."""
    if os.environ.get(_FAMILY_ENV_FLAG, "1") == "0":
        return False
    if os.environ.get(_ROPE_ENV_FLAG, "1") == "0":
        return False
    return _metal_available()


def prefill_rope_seam_enabled() -> bool:
    """True when prefill row counts may use the fused launch (reference :150)."""
    return os.environ.get(_PREFILL_ENV_FLAG, "1") != "0"


def _element_dtypes():
    return (torch.float32, torch.float16, torch.bfloat16)


def partial_rope_eligible(x, inv_freq, *, offset, positions) -> bool:
    """The DS4 rope contract (reference :200-244); every miss answers False."""
    if not isinstance(x, torch.Tensor) or x.ndim < 2 or x.dtype not in _element_dtypes():
        return False
    width = int(x.shape[-1])
    if width < _ROPE_DIM or width % 4 != 0:
        return False
    seq_len = int(x.shape[-2])
    rows = 1
    for dim in x.shape[:-1]:
        rows *= int(dim)
    max_rows = _MAX_ROWS_PREFILL if prefill_rope_seam_enabled() else _MAX_ROWS_DECODE
    if not 1 <= rows <= max_rows:
        return False
    if (not isinstance(inv_freq, torch.Tensor) or inv_freq.ndim != 1 or int(inv_freq.shape[0]) != _ROPE_FREQS
            or inv_freq.dtype != torch.float32):
        return False
    if positions is None:
        if not isinstance(offset, int) or isinstance(offset, bool):
            return False
        if offset < 0 or offset + seq_len > _MAX_EXACT_POSITION:
            return False
        return True
    if not isinstance(positions, torch.Tensor):
        return False
    if positions.dtype != torch.float32 or positions.numel() != seq_len:
        return False
    return True


def fused_partial_rope(x, inv_freq, *, offset=0, inverse=False, positions=None):
    """Apply the DS4 partial rope in one launch (reference :247).

    Args:
        x: ``[..., seq, width]`` float32, float16, or bfloat16 rows; the final 64 channels rotate
            (interleaved pairs), the leading channels copy through.
        inv_freq: float32 ``[32]`` rope inverse frequencies (YaRN folded).
        offset: absolute position of the first sequence row; used when ``positions`` is None.
        inverse: negate the rotation.
        positions: optional float32 positions for the sequence axis.

    Returns:
        A tensor of the same shape and dtype.
    """
    if not partial_rope_eligible(x, inv_freq, offset=offset, positions=positions):
        raise ValueError("operands are outside the fused partial-rope contract")
    _lib.require_device(x, inv_freq, positions)
    width = int(x.shape[-1])
    seq_len = int(x.shape[-2])
    rows = x.numel() // width
    xc = x.contiguous()
    out = torch.empty_like(xc)
    inv = inv_freq.contiguous()
    pos = None if positions is None else positions.reshape(seq_len).contiguous()
    form = "off" if positions is None else "pos"
    dtype_code = _lib.DTYPE_CODE[x.dtype]
    rc = _lib.lib().mspr_fused_partial_rope(_lib.ptr(xc), dtype_code, rows // seq_len, seq_len, width, _lib.ptr(inv),
                                            _lib.ptr(pos), 0 if positions is not None else int(offset),
                                            1 if inverse else 0, _lib.ptr(out), _lib.stream_ptr())
    _lib.check(rc, "fused_partial_rope")
    _ROPE_KERNELS[(form, bool(inverse))] = f"mspr_fused_partial_rope[{form},{'inv' if inverse else 'fwd'}]"
    return out.reshape(x.shape)
