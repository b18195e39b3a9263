"""GPU parity of the entry point that allocates nothing (static scratch inside the library) against the
workspace form of the same operator, through the C-ABI: two calls in a row, the second smaller."""

import numpy as np
import pytest
import torch

from moespresso_amd import _lib

pytestmark = pytest.mark.gpu


def _call(static, q, kv, ids, sinks, win_rows, ws=None):
    B, H, DK = q.shape
    N = kv.shape[1]
    out = torch.empty((B, H, 512), dtype=q.dtype, device=q.device)
    common = [_lib.ptr(q), _lib.ptr(kv), _lib.ptr(ids), _lib.ptr(sinks), _lib.DTYPE_CODE[q.dtype], B, H, DK, 512, N,
              int(ids.shape[1]), 4, 3, N - win_rows, win_rows, float(DK ** -0.5), _lib.ptr(out)]
    if static:
        rc = _lib.lib().mspr_sparse_mla_decode_static(*common, _lib.stream_ptr())
    else:
        rc = _lib.lib().mspr_sparse_mla_decode(*common, _lib.ptr(ws), ws.numel() * 4, _lib.stream_ptr())
    _lib.check(rc, "sparse_mla_decode")
    return out


def _inputs(B, H, N, R, seed):
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(seed)
    kv = torch.randn((B, N, 576), device=dev, generator=gen).to(torch.bfloat16)
    q = torch.randn((B, H, 576), device=dev, generator=gen).to(torch.bfloat16)
    rng = np.random.default_rng(seed)
    ids = np.stack([np.sort(rng.choice((N - 128) // 4, R, replace=False)) for _ in range(B)]).astype(np.int32)
    sinks = torch.randn((H,), device=dev, generator=gen)
    return q, kv, torch.from_numpy(ids).to(dev), sinks


def test_static_scratch_entry_matches_workspace_entry_twice():
    dev = torch.device("cuda:0")
    # first call: 16 sequences x 16 key ranges (all 256 partial slots of the scratch); second: smaller in
    # batch, heads and rows, so other range counts and counters are used on the same scratch
    for (B, H, N, R, seed) in ((16, 64, 16384, 2048, 1), (3, 40, 4096, 301, 2)):
        q, kv, ids, sinks = _inputs(B, H, N, R, seed)
        ws = _lib.sparse_attention_workspace(B, H, R + 128, dev)
        want = _call(False, q, kv, ids, sinks, 128, ws)
        got = _call(True, q, kv, ids, sinks, 128)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (B, H, N, R)
        assert torch.isfinite(got.float()).all()


def test_static_scratch_entry_rejects_what_does_not_fit():
    q, kv, ids, sinks = _inputs(2, 64, 4096, 16, 5)
    big_rows = torch.zeros((2, 200000), dtype=torch.int32, device=q.device)
    out = torch.empty((2, 64, 512), dtype=q.dtype, device=q.device)
    rc = _lib.lib().mspr_sparse_mla_decode_static(
        _lib.ptr(q), _lib.ptr(kv), _lib.ptr(big_rows), _lib.ptr(sinks), 2, 2, 64, 576, 512, 4096, 200000, 4, 3,
        4096 - 128, 128, float(576 ** -0.5), _lib.ptr(out), _lib.stream_ptr())
    assert rc == _lib.MSPR_ERR_ARG
    assert b"scratch" in _lib.lib().mspr_last_error()
    assert int(_lib.lib().mspr_sparse_mla_decode_static_max_bytes()) == 256 * (64 * 512 * 2 + 64 * 2 * 4)
