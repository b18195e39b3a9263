"""ctypes binding of libmoespresso_amd.so (the C-ABI in include/moespresso_amd.h).

The library is loaded lazily and only from this package directory. There is no
fallback: a missing library or a tensor that is not on a HIP device raises.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmoespresso_amd.so")

MSPR_OK = 0
MSPR_ERR_ARG = -1
MSPR_ERR_LAUNCH = -2

DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

# name -> (restype, argtypes); one entry per symbol declared in include/moespresso_amd.h
SIGNATURES = {
    "mspr_abi_version": (c_int, []),
    "mspr_last_error": (c_char_p, []),
    "mspr_indexer_qat_rows": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_void_p]),
    "mspr_fused_qat_indexer_scores": (
        c_int, [c_void_p, c_int, c_int, c_void_p, c_int64, c_void_p, c_float, c_void_p, c_void_p]),
    "mspr_indexer_score_tail": (
        c_int, [c_void_p, c_int, c_int64, c_void_p, c_int, c_void_p, c_float, c_void_p, c_void_p]),
    "mspr_fp8_kv_prefix_rows": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "mspr_topk_select": (c_int, [c_void_p, c_int64, c_int, c_int64, c_int, c_void_p, c_void_p]),
    "mspr_fused_decode_prep": (
        c_int, [c_void_p, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                c_float, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "mspr_fused_decode_prep_fixed": (
        c_int, [c_void_p, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                c_float, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "mspr_fused_decode_sdpa_fixed": (
        c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int64, c_void_p, c_int, c_void_p,
                c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_size_t, c_void_p]),
    "mspr_indexer_scores_fp8": (
        c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_void_p, c_void_p]),
    "mspr_indexer_q_qat_live": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "mspr_indexer_scores_tiled_live": (
        c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int64, c_int64, c_int, c_void_p,
                c_void_p]),
    "mspr_indexed_mixed_attention_prefill": (
        c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p, c_int64,
                c_void_p, c_int, c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "mspr_sparse_attention_workspace_bytes": (c_size_t, [c_int, c_int, c_int64]),
    "mspr_indexed_mixed_attention_prefill_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "mspr_indexed_mixed_attention_decode": (
        c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int64, c_void_p, c_int, c_void_p, c_int64,
                c_int, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "mspr_fused_decode_sdpa": (
        c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int64, c_void_p, c_int, c_void_p,
                c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_size_t, c_void_p]),
    "mspr_sparse_mla_decode": (
        c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int64, c_int,
                c_int, c_int, c_int64, c_int, c_float, c_void_p, c_void_p, c_size_t, c_void_p]),
    "mspr_sparse_mla_decode_static": (
        c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int64, c_int,
                c_int, c_int, c_int64, c_int, c_float, c_void_p, c_void_p]),
    "mspr_sparse_mla_decode_static_max_bytes": (c_size_t, []),
    "mspr_fused_partial_rope": (
        c_int, [c_void_p, c_int, c_int64, c_int64, c_int, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p]),
    "mspr_affine_q8_quantize": (
        c_int, [c_void_p, c_int, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "mspr_affine_q8_dequantize": (
        c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_void_p, c_int, c_int, c_void_p]),
    "mspr_sdpa_decode_q8_workspace_bytes": (c_size_t, [c_int, c_int, c_int64]),
    "mspr_sdpa_decode_q8": (
        c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                c_int, c_int, c_int64, c_int64, c_float, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "mspr_sdpa_decode_q8_0": (
        c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int64,
                c_int64, c_float, c_void_p, c_void_p, c_size_t, c_void_p]),
    "mspr_flash_prefill": (
        c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int64, c_int64, c_float,
                c_void_p, c_void_p, c_size_t, c_void_p]),
    "mspr_flash_prefill_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int64]),
    "mspr_sdpa_fa_prefill_q8_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int64]),
    "mspr_sdpa_fa_prefill_q8": (
        c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                c_int, c_int, c_int, c_int, c_int, c_int, c_int64, c_int64, c_float, c_int, c_int, c_void_p, c_void_p,
                c_size_t, c_void_p]),
    "mspr_profile_enable": (c_int, [c_int]),
    "mspr_profile_collect": (c_int, [c_int, c_void_p, c_int]),
}

# kernel ids of mspr_profile_enable / mspr_profile_collect
KERNEL_IDS = {"indexer_fp8": 1, "topk": 2, "sparse_split": 3, "sparse_merge": 4, "scores_f32": 5,
              "q8_decode": 6, "q8_merge": 7, "flash_prefill": 8}


def profile_enable(*names: str) -> None:
    """Bracket later launches of the named kernels with HIP events (no names = off)."""
    mask = 0
    for n in names:
        mask |= 1 << KERNEL_IDS[n]
    lib().mspr_profile_enable(mask)


def profile_collect(name: str, max_n: int = 65536) -> list[float]:
    """Durations (ms) of the recorded launches of one kernel; waits for them and clears them."""
    buf = (ctypes.c_float * max_n)()
    n = lib().mspr_profile_collect(KERNEL_IDS[name], ctypes.cast(buf, c_void_p), max_n)
    return [float(buf[i]) for i in range(n)]


def sparse_attention_workspace(batch: int, n_heads: int, n_keys: int, device) -> torch.Tensor:
    """Scratch tensor for the gathered-attention entry points (split partials)."""
    nbytes = int(lib().mspr_sparse_attention_workspace_bytes(int(batch), int(n_heads), int(n_keys)))
    return torch.empty((max(nbytes, 16) + 3) // 4, dtype=torch.float32, device=device)


def prefill_attention_workspace(q_dtype, batch: int, n_heads: int, n_tokens: int, window_rows: int, top_k: int,
                                device) -> torch.Tensor:
    """Scratch tensor for mspr_indexed_mixed_attention_prefill (split partials, or the half copy of float32 queries)."""
    nbytes = int(lib().mspr_indexed_mixed_attention_prefill_workspace_bytes(
        DTYPE_CODE[q_dtype], int(batch), int(n_heads), int(n_tokens), int(window_rows), int(top_k)))
    return torch.empty((max(nbytes, 16) + 3) // 4, dtype=torch.float32, device=device)


def q8_decode_workspace(batch: int, n_kv_heads: int, n_keys: int, device) -> torch.Tensor:
    """Scratch tensor for the Q8 decode entry points (per-range partials)."""
    nbytes = int(lib().mspr_sdpa_decode_q8_workspace_bytes(int(batch), int(n_kv_heads), int(n_keys)))
    return torch.empty((max(nbytes, 16) + 3) // 4, dtype=torch.float32, device=device)


_LIB = None


def library_available() -> bool:
    """True when the shared library exists on disk (it is not loaded here)."""
    return os.path.exists(LIB_PATH)


def lib() -> ctypes.CDLL:
    """Load (once) and return the shared library; raises if it was never built."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m moespresso_amd.build` "
                "(there is no CPU or PyTorch fallback for these operators)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _LIB = handle
    return _LIB


def hip_available() -> bool:
    """True when a HIP device is visible and the kernel library is present."""
    return bool(torch.cuda.is_available()) and library_available()


def check(rc: int, what: str) -> None:
    """Map a C-ABI return code to a Python exception."""
    if rc == MSPR_OK:
        return
    msg = lib().mspr_last_error().decode("utf-8", "replace")
    if rc == MSPR_ERR_ARG:
        raise ValueError(f"{what}: {msg}")
    raise RuntimeError(f"{what}: {msg}")


def require_device(*tensors: torch.Tensor) -> torch.device:
    """All tensors must live on one HIP device; returns it."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "moespresso_amd operators run on a HIP device only; got a tensor on "
                f"{t.device} (there is no CPU fallback)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("all operands must be on the same HIP device")
    return dev


def ptr(t: torch.Tensor | None) -> c_void_p:
    if t is None:
        return c_void_p(0)
    return c_void_p(t.data_ptr())


def stream_ptr() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)
