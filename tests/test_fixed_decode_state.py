"""Fixed-capacity decode state: the capacity-buffer bookkeeping on CPU tensors (reference
fixed_decode_state.py:186-288) and, on the GPU, one HIP graph of the fused decode island replayed while the
pool grows, against eager calls on the growing layout."""

import numpy as np
import pytest
import torch

from moespresso_amd.runtime.deepseek_v4 import fixed_decode_state as fds
from oracle import ds4


def test_aux_fixed_update_appends_adopts_and_fails_closed(monkeypatch):
    calls = []

    def transform(rows):
        calls.append(int(rows.shape[1]))
        return rows.float() * 2.0

    branch = fds._FixedBranchState(ratio=4, max_context=64)           # 16 rows of capacity
    assert branch.pool_capacity == 16 and fds.aux_capacity_buffer(branch, "pooled_qat") is None
    state = {}
    pool = torch.arange(16 * 3, dtype=torch.float16).reshape(1, 16, 3)
    view, prior = fds.aux_fixed_update(branch, state, name="pooled_qat", rows_key="pooled_qat_rows",
                                       pooled=pool[:, :5], transform=transform)
    assert prior == 0 and calls == [5] and tuple(view.shape) == (1, 5, 3) and state["pooled_qat"] is view
    cap = fds.aux_capacity_buffer(branch, "pooled_qat")
    assert tuple(cap.shape) == (1, 16, 3) and cap.dtype == torch.float32 and state["pooled_qat_rows"] == 5
    # one more row: only the tail is transformed, into the same buffer
    view2, prior = fds.aux_fixed_update(branch, state, name="pooled_qat", rows_key="pooled_qat_rows",
                                        pooled=pool[:, :6], transform=transform)
    assert prior == 5 and calls == [5, 1] and fds.aux_capacity_buffer(branch, "pooled_qat") is cap
    assert view2.data_ptr() == cap.data_ptr() and torch.equal(view2, pool[:, :6].float() * 2.0)
    # unchanged pool: nothing to do
    _, prior = fds.aux_fixed_update(branch, state, name="pooled_qat", rows_key="pooled_qat_rows", pooled=pool[:, :6],
                                    transform=transform)
    assert prior == 6 and calls == [5, 1]
    # a legacy key replaced behind the buffer's back is adopted (it is authoritative)
    state["pooled_qat"] = torch.full((1, 4, 3), 7.0)
    state["pooled_qat_rows"] = 4
    view3, prior = fds.aux_fixed_update(branch, state, name="pooled_qat", rows_key="pooled_qat_rows",
                                        pooled=pool[:, :6], transform=transform)
    assert prior == 4 and calls == [5, 1, 2] and torch.equal(view3[:, :4], torch.full((1, 4, 3), 7.0))
    # fail closed: capacity exceeded, malformed legacy cache, element type change
    big = torch.zeros((1, 17, 3), dtype=torch.float16)
    assert fds.aux_fixed_update(branch, state, name="pooled_qat", rows_key="pooled_qat_rows", pooled=big,
                                transform=transform) is None
    bad = {"x": torch.zeros((1, 3, 3)), "x_rows": 9}
    assert fds.aux_fixed_update(branch, bad, name="x", rows_key="x_rows", pooled=pool[:, :10], transform=transform) is None
    assert fds.aux_fixed_update(branch, state, name="pooled_qat", rows_key="pooled_qat_rows", pooled=pool[:, :8],
                                transform=lambda r: r.double()) is None
    # env knobs are read per call
    monkeypatch.setenv("MOESPRESSO_DSV4_DECODE_MAX_CONTEXT", "1000")
    assert fds.fixed_decode_max_context() == 1000 and fds._FixedBranchState(ratio=4).pool_capacity == 250
    monkeypatch.setenv("MOESPRESSO_DSV4_DECODE_FIXED_STATE", "0")
    assert not fds.fixed_decode_state_enabled()


@pytest.mark.gpu
def test_one_graph_serves_consecutive_tokens_while_the_pool_grows():
    from moespresso_amd import _lib
    from moespresso_amd.runtime.deepseek_v4 import decode_attention_kernel as dak
    from moespresso_amd.runtime.deepseek_v4 import indexer_score_kernel as isk

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(3)
    cap, topk, H, W = 1024, 64, 64, 128
    inv = torch.from_numpy(ds4.rope_inverse_frequencies(64, ds4.DS4_COMPRESS_ROPE_BASE, ds4.DS4_YARN).astype(np.float32)).to(dev)
    branch = fds._FixedBranchState(ratio=4, pool_capacity=cap)
    pool_idx = torch.randn((1, cap, 128), device=dev, generator=g)            # indexer pool, as the compressor grows it
    pooled_cap = torch.zeros((cap, 512), dtype=torch.float16, device=dev)     # attention pool, capacity layout
    pool_rows_all = (torch.randn((cap, 512), device=dev, generator=g) * 0.1).half()
    state = {}
    # persistent operands of the captured step
    q_idx = torch.zeros((H, 128), device=dev)
    weights = torch.zeros((H,), device=dev)
    kv_row = torch.zeros((512,), dtype=torch.float16, device=dev)
    q = torch.zeros((H, 512), dtype=torch.float16, device=dev)
    window = (torch.randn((W, 512), device=dev, generator=g) * 0.1).half()
    sinks = torch.randn((H,), device=dev, generator=g).half()
    params = fds.DecodeStepParams(dev)
    ws = _lib.sparse_attention_workspace(1, H, W + topk, dev)

    def refresh(rows):
        view, _ = fds.aux_fixed_update(branch, state, name="pooled_qat", rows_key="pooled_qat_rows",
                                       pooled=pool_idx[:, :rows], transform=isk.indexer_qat_rows)
        pooled_cap[:rows] = pool_rows_all[:rows]
        q_idx.copy_(torch.randn((H, 128), device=dev, generator=g))
        weights.copy_(torch.rand((H,), device=dev, generator=g) * H ** -0.5)
        kv_row.copy_((torch.randn((512,), device=dev, generator=g) * 0.2).half())
        q.copy_((torch.randn((H, 512), device=dev, generator=g) * 0.1).half())
        return view

    def island():
        qat_cap = fds.aux_capacity_buffer(branch, "pooled_qat")[0]
        sel, row, scores = dak.fused_decode_prep(q_idx, qat_cap, weights, kv_row, inv, params.tensor, scale=128 ** -0.5,
                                                 topk=topk, pool_rows_in_params=True)
        out = dak.fused_decode_sdpa(q, window, row, pooled_cap, sel, sinks, inv, params.tensor, scale=512 ** -0.5,
                                    pool_rows_in_params=True, workspace=ws)
        return sel, row, scores, out

    rows, offset, widx = 300, 4000, 17
    refresh(rows)
    params.set(offset=offset, write_idx=widx, pool_rows=rows)
    island()                                                    # loads the code objects before capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sel_g, row_g, scores_g, out_g = island()
    for step in range(6):
        rows += (1, 0, 3, 0, 40, 1)[step]                       # the pool gains rows on some tokens only
        offset, widx = offset + 1, (widx + 1) % W
        qat_view = refresh(rows)
        params.set(offset=offset, write_idx=widx, pool_rows=rows)
        graph.replay()
        torch.cuda.synchronize()
        # eager, growing layout: the first `rows` rows as tensors of their own, params without a row count
        p2 = torch.tensor([offset, widx], dtype=torch.int32, device=dev)
        sel, row, scores = dak.fused_decode_prep(q_idx, qat_view[0].contiguous(), weights, kv_row, inv, p2,
                                                 scale=128 ** -0.5, topk=topk)
        out = dak.fused_decode_sdpa(q, window, row, pooled_cap[:rows].contiguous(), sel, sinks, inv, p2,
                                    scale=512 ** -0.5)
        torch.cuda.synchronize()
        assert torch.equal(sel_g, sel) and torch.equal(row_g, row), step
        assert torch.equal(scores_g[:rows], scores) and bool(torch.isneginf(scores_g[rows:]).all()), step
        assert torch.equal(out_g, out), step
        window[widx] = row                                      # the ring append the wrapper does after the island


@pytest.mark.gpu
def test_fewer_rows_in_use_than_the_selection_width():
    from moespresso_amd.runtime.deepseek_v4 import decode_attention_kernel as dak

    dev = torch.device("cuda:0")
    rng = np.random.default_rng(12)
    cap, topk, H, rows = 256, 64, 16, 20
    inv = ds4.rope_inverse_frequencies(64, ds4.DS4_COMPRESS_ROPE_BASE, ds4.DS4_YARN).astype(np.float32)
    qat = ds4.indexer_qat(rng.standard_normal((cap, 128)).astype(np.float32))
    pooled = (rng.standard_normal((cap, 512)) * 0.1).astype(np.float16)
    q_idx = rng.standard_normal((H, 128)).astype(np.float32)
    w = (rng.uniform(0, 1, H) * H ** -0.5).astype(np.float32)
    kv = (rng.standard_normal(512) * 0.2).astype(np.float16)
    q = (rng.standard_normal((H, 512)) * 0.1).astype(np.float16)
    window = (rng.standard_normal((128, 512)) * 0.1).astype(np.float16)
    sinks = rng.standard_normal(H).astype(np.float16)
    params = np.array([900, 5, rows], np.int32)
    t = lambda a: torch.from_numpy(a).to(dev)
    sel, row, scores = dak.fused_decode_prep(t(q_idx), t(qat), t(w), t(kv), t(inv), t(params), scale=128 ** -0.5,
                                             topk=topk, pool_rows_in_params=True)
    sel_h = sel.cpu().numpy()
    assert sorted(sel_h[sel_h < rows].tolist()) == list(range(rows))      # every row in use is selected
    np.testing.assert_array_equal(sel_h[rows:], np.arange(rows, topk))    # then unused rows, all tied at -inf
    out = dak.fused_decode_sdpa(t(q), t(window), row, t(pooled), sel, t(sinks), t(inv), t(params), scale=512 ** -0.5,
                                pool_rows_in_params=True)
    want = ds4.fused_decode_sdpa(q, window, row.cpu().numpy(), pooled[:rows], sel_h[:rows], sinks, inv, params[:2],
                                 scale=512 ** -0.5)
    assert np.abs(out.float().cpu().numpy() - want.astype(np.float32)).max() < 2e-3
