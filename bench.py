#!/usr/bin/env python
"""Benchmark of the MI355X attention hot path.

One step = one DeepSeek-V4-style sparse decode attention layer at 128K context on synthetic data:

    lightning-indexer scores (64 heads x 128, 32768 fp8 keys per sequence)
      -> deterministic top-2048
      -> sparse multi-head-latent decode attention over the 2048 gathered rows plus the last
         128 rows of a 131072-token bf16 latent cache (576-wide K, 512-wide V, 64 heads)

for a batch of 16 sequences (BASELINE configs 4 and 5 chained). Inputs are resident in HBM before
the timed region; the step is captured in a HIP graph per buffer set and the timed loop replays
the graphs round-robin over several buffer sets so that neither L2 nor the Infinity Cache can hold
the streamed rows between steps.

Prints ONE JSON line (see README of the driver contract): metric/value plus `roofline` for the
dominant kernel (GPU-side duration from HIP events around that kernel on its launch stream) and
`cpu_baseline` (a threaded torch restatement of the same layer, pinned against the NumPy oracle by the
CPU tests, on a bounded sample on this host's cores; the float64 NumPy oracle itself is timed beside it).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0  # dense bf16 / f16
COUNTERS_FILE = os.path.join(ROOT, "profiles", "bench_sparse_decode_layer_hbm_counters.txt")
TRACE_FILE = os.path.join(ROOT, "profiles", "bench_all_kernels_kernel_trace_stats.txt")
SPLIT_KERNEL_SOURCE = os.path.join(ROOT, "moespresso_amd", "csrc", "sparse_attn.hip")


def host_threads() -> int:
    """Threads the CPU legs use: the host's cores, at most 16 (the CPU share of a one-GPU box)."""
    return min(16, os.cpu_count() or 1)


def source_sha256(path: str = SPLIT_KERNEL_SOURCE) -> str | None:
    import hashlib

    try:
        with open(path, "rb") as f:
            return hashlib.sha256(f.read()).hexdigest()
    except OSError:
        return None


def profile_is_current(path: str) -> bool:
    """A committed rocprofv3 summary records the SHA-256 of the kernel source it was taken from (a line
    `source_sha256 sparse_attn.hip <hex>`); figures from it are reported only while that source is unchanged."""
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("source_sha256 sparse_attn.hip"):
                    return line.split()[-1] == source_sha256()
    except OSError:
        pass
    return False


def traced_kernel_us(kernel_prefix: str, workgroups: str):
    """Average duration (us) of one kernel and launch shape (`workgroups` as "256x1x1") in the committed
    `rocprofv3 --kernel-trace --stats` summary of this benchmark (graph-replayed launches: no event records around
    the kernel), or None."""
    import re

    if not profile_is_current(TRACE_FILE):
        return None
    row = re.compile(r"^(?P<name>.+?)\s+(?P<wg>\d+x\d+x\d+)\s+\d+\s+\d+\s+(?P<avg>[\d.]+)\s+[\d.]+\s+[\d.]+\s*$")
    try:
        with open(TRACE_FILE) as f:
            for line in f:
                m = row.match(line)
                if m and m.group("name").startswith(kernel_prefix) and m.group("wg") == workgroups:
                    return float(m.group("avg"))
    except (OSError, ValueError):
        pass
    return None


def measured_traffic_bytes(kernel_prefix: str, workgroups: int):
    """HBM bytes per launch of one kernel as the committed rocprofv3 counter summary reports them (FETCH_SIZE +
    WRITE_SIZE, each scaled by the same counter's reading for a copy kernel of known size); None when the
    summary does not hold that launch shape."""
    if not profile_is_current(COUNTERS_FILE):
        return None
    try:
        with open(COUNTERS_FILE) as f:
            for line in f:
                if not line.startswith(kernel_prefix):
                    continue
                cols = line[44:].split()
                if len(cols) >= 7 and int(cols[0]) == workgroups:
                    return int(round(float(cols[6]) * 1e6))
    except (OSError, ValueError):
        pass
    return None

# workload constants (BASELINE configs 4 and 5)
N_IDX_HEADS, IDX_DIM, N_KEYS, TOPK = 64, 128, 32768, 2048
N_HEADS, K_DIM, V_DIM, N_TOKENS, WINDOW = 64, 576, 512, 131072, 128
# algorithmic bytes per sequence: gathered rows + q + out + ids (config 5); keys + scales + q,w + ids (config 4)
MLA_BYTES_PER_SEQ = (TOPK + WINDOW) * K_DIM * 2 + N_HEADS * K_DIM * 2 + N_HEADS * V_DIM * 2 + TOPK * 4
IDX_BYTES_PER_SEQ = N_KEYS * IDX_DIM + N_KEYS * 4 + N_IDX_HEADS * IDX_DIM * 2 + N_IDX_HEADS * 4 + TOPK * 4


def make_set(batch: int, dev, gen):
    qi = torch.randn((batch, N_IDX_HEADS, IDX_DIM), device=dev, generator=gen).to(torch.bfloat16)
    k32 = torch.randn((batch, N_KEYS, IDX_DIM), device=dev, generator=gen)
    kscale = (k32.abs().amax(dim=-1) / 448.0).contiguous()
    keys = (k32 / kscale[..., None]).to(torch.float8_e4m3fn)
    del k32
    w = torch.rand((batch, N_IDX_HEADS), device=dev, generator=gen)
    q = torch.randn((batch, N_HEADS, K_DIM), device=dev, generator=gen).to(torch.bfloat16)
    kv = torch.empty((batch, N_TOKENS, K_DIM), device=dev, dtype=torch.bfloat16)
    for b in range(batch):  # chunked: the float32 intermediate of one sequence is 302 MB
        kv[b] = torch.randn((N_TOKENS, K_DIM), device=dev, generator=gen).to(torch.bfloat16)
    return dict(qi=qi, keys=keys, kscale=kscale, w=w, q=q, kv=kv)


def cpu_baseline_torch(seconds_budget: float = 10.0, threads: int | None = None):
    """The torch restatement of the layer (oracle/ds4_torch.py, float32, threaded) on one sequence of the same
    step, scaled to the 16-sequence layer."""
    from oracle import ds4_torch

    cores = host_threads() if threads is None else threads
    before = torch.get_num_threads()
    torch.set_num_threads(cores)
    try:
        g = torch.Generator().manual_seed(0)
        qi = torch.randn((N_IDX_HEADS, IDX_DIM), generator=g).to(torch.bfloat16).float()
        k32 = torch.randn((N_KEYS, IDX_DIM), generator=g)
        kscale = k32.abs().amax(dim=-1) / 448.0
        codes = (k32 / kscale[:, None]).to(torch.float8_e4m3fn).view(torch.uint8)
        w = torch.rand((N_IDX_HEADS,), generator=g)
        q = torch.randn((N_HEADS, K_DIM), generator=g).to(torch.bfloat16).float()
        kv = torch.randn((N_TOKENS, K_DIM), generator=g).to(torch.bfloat16)

        def step():
            return ds4_torch.decode_layer(qi, codes, kscale, w, q, kv, topk=TOPK, window=WINDOW, scale=K_DIM ** -0.5)

        step()
        t0 = time.perf_counter()
        reps = 0
        while reps < 200 and (time.perf_counter() - t0) < seconds_budget:
            step()
            reps += 1
        per_seq = (time.perf_counter() - t0) / max(reps, 1)
    finally:
        torch.set_num_threads(before)
    return {
        "value": round(per_seq * 16 * 1e6, 1),
        "unit": "us/layer",
        "cores": cores,
        "host_cpus": os.cpu_count(),
        "kind": "port",
        "sample": f"{reps} repeats of one sequence (1/16 of the layer: 32768-key indexer + top-2048 + 2176-row "
                  f"MLA decode), torch float32 restatement of the layer with {cores} threads, scaled x16",
    }


def cpu_baseline(seconds_budget: float = 10.0, threads: int | None = None):
    """The NumPy oracle on one sequence of the same step; scaled to the 16-sequence layer."""
    from oracle import ds4

    try:
        from threadpoolctl import threadpool_limits
    except Exception:  # pragma: no cover
        threadpool_limits = None
    cores = host_threads() if threads is None else threads
    rng = np.random.default_rng(0)
    qi = ds4.round_bf16(rng.standard_normal((1, N_IDX_HEADS, IDX_DIM), dtype=np.float32))
    k32 = rng.standard_normal((1, N_KEYS, IDX_DIM), dtype=np.float32)
    kscale = (np.abs(k32).max(-1) / 448.0).astype(np.float32)
    codes = ds4.e4m3_encode(k32 / kscale[..., None])
    w = rng.uniform(0, 1, (1, N_IDX_HEADS)).astype(np.float32)
    q = ds4.round_bf16(rng.standard_normal((1, N_HEADS, K_DIM), dtype=np.float32))
    kv = ds4.round_bf16(rng.standard_normal((1, N_TOKENS, K_DIM), dtype=np.float32))
    win = np.arange(N_TOKENS - WINDOW, N_TOKENS, dtype=np.int64)

    def step():
        s = ds4.indexer_scores_fp8(qi, codes, kscale, w)
        sel = ds4.radix_select_topk(s[0].astype(np.float32), TOPK).astype(np.int64)
        rows = np.concatenate([win, 4 * sel + 3])[None, :]
        return ds4.sparse_mla_decode(q, kv, rows, scale=K_DIM ** -0.5)

    ctx = threadpool_limits(limits=cores) if threadpool_limits else None
    try:
        step()
        t0 = time.perf_counter()
        reps = 0
        while reps < 20 and (time.perf_counter() - t0) < seconds_budget:
            step()
            reps += 1
        per_seq = (time.perf_counter() - t0) / max(reps, 1)
    finally:
        if ctx is not None:
            ctx.__exit__(None, None, None)
    return {
        "value": per_seq * 16 * 1e6,
        "unit": "us/layer",
        "cores": cores,
        "kind": "port",
        "sample": f"{reps} repeats of one sequence (1/16 of the layer: 32768-key indexer + top-2048 + 2176-row "
                  f"MLA decode), float64 NumPy oracle with {cores} BLAS threads (its time is the float64 score "
                  f"sum and the selection, which no BLAS call covers), scaled x16",
    }


def cpu_other_configs():
    """BASELINE configs 2 and 3 on the host through the NumPy oracle, on bounded samples (a reported baseline):
    config 3 whole at batch 1; config 2 on 128 of the 4096 query rows (the last ones: the deepest causal rows),
    scaled by the ratio of causal FLOPs."""
    from oracle import qwen

    try:
        from threadpoolctl import threadpool_limits
    except Exception:  # pragma: no cover
        threadpool_limits = None
    cores = host_threads()
    rng = np.random.default_rng(0)
    out = {}
    ctx = threadpool_limits(limits=cores) if threadpool_limits else None
    try:
        N = 37000
        kc, ks = qwen.q8_0_quantize(rng.standard_normal((1, 2, N, 256), dtype=np.float32))
        vc, vs = qwen.q8_0_quantize(rng.standard_normal((1, 2, N, 256), dtype=np.float32))
        q = rng.standard_normal((1, 16, 1, 256), dtype=np.float32)

        def decode():
            return qwen.gqa_decode_attention(q, qwen.q8_0_dequantize(kc, ks), qwen.q8_0_dequantize(vc, vs), 256 ** -0.5)

        t0 = time.perf_counter()
        decode()
        reps = 1
        if time.perf_counter() - t0 < 1.0:  # fast host: the first call was the warm-up
            t0 = time.perf_counter()
            reps = 0
            while reps < 20 and time.perf_counter() - t0 < 3.0:
                decode()
                reps += 1
        out["config3_B1_us"] = round((time.perf_counter() - t0) / max(reps, 1) * 1e6, 1)
        out["config3_sample"] = f"{reps} repeats, dequantise + float64 attention over 37000 keys, batch 1"
        L, past, rows = 4096, 32768, 128
        k = (0.5 * rng.standard_normal((1, 2, past + L, 256), dtype=np.float32))
        v = (0.5 * rng.standard_normal((1, 2, past + L, 256), dtype=np.float32))
        qs = (0.5 * rng.standard_normal((1, 16, rows, 256), dtype=np.float32))
        t0 = time.perf_counter()
        qwen.causal_prefill_attention(qs, k, v, 256 ** -0.5, past=past + L - rows)
        dt = time.perf_counter() - t0
        sample_flops = 4.0 * 256 * 16 * sum(past + L - rows + i + 1 for i in range(rows))
        full_flops = 4.0 * 256 * 16 * (L * past + L * (L + 1) / 2)
        out["config2_ms"] = round(dt * full_flops / sample_flops * 1e3, 1)
        out["config2_sample"] = f"the last {rows} of {L} query rows once ({dt:.2f} s), scaled by causal FLOPs x{full_flops / sample_flops:.1f}"
    finally:
        if ctx is not None:
            ctx.__exit__(None, None, None)
    out["cores"] = cores
    out["kind"] = "port"
    return out


def cpu_config1():
    """BASELINE config 1 (dense GQA decode, 8 q heads / 1 KV head, D=128, 4096 keys, fp16) on the host: the NumPy
    restatement of softmax attention, warm-up 3, 20 repeats."""
    from oracle import qwen

    rng = np.random.default_rng(0)
    q = rng.standard_normal((1, 8, 1, 128)).astype(np.float16)
    k = rng.standard_normal((1, 1, 4096, 128)).astype(np.float16)
    v = rng.standard_normal((1, 1, 4096, 128)).astype(np.float16)
    for _ in range(3):
        qwen.gqa_decode_attention(q, k, v, 128 ** -0.5)
    t0 = time.perf_counter()
    for _ in range(20):
        qwen.gqa_decode_attention(q, k, v, 128 ** -0.5).astype(np.float16)
    return {"us": round((time.perf_counter() - t0) / 20 * 1e6, 1), "kind": "port", "cores": 1,
            "workload": "dense GQA decode, 8q/1kv heads, D=128, 4096 fp16 keys (BASELINE config 1), NumPy float64"}


def bench_prefill(dev, gen, reps=10, warmup=20):
    """BASELINE config 2: 4096-token bf16 chunk over a 32768-token prefix, 16 q / 2 KV heads, D=256.

    The launches run back to back; the first ones after lighter work are about a tenth slower than the
    sustained rate, hence the warm-up."""
    from moespresso_amd import _lib
    from moespresso_amd.runtime.qwen import kquant

    L, past = 4096, 32768
    q = (0.5 * torch.randn((1, 16, L, 256), device=dev, generator=gen)).to(torch.bfloat16)
    k = (0.5 * torch.randn((1, 2, past + L, 256), device=dev, generator=gen)).to(torch.bfloat16)
    v = (0.5 * torch.randn((1, 2, past + L, 256), device=dev, generator=gen)).to(torch.bfloat16)
    for _ in range(warmup):
        kquant.flash_prefill(q, k, v, 256 ** -0.5, past_len=past)
    torch.cuda.synchronize()
    _lib.profile_enable("flash_prefill")
    for _ in range(reps):
        kquant.flash_prefill(q, k, v, 256 ** -0.5, past_len=past)
    torch.cuda.synchronize()
    ms = float(np.mean(_lib.profile_collect("flash_prefill")))
    _lib.profile_enable()
    flops = 4.0 * 256 * 16 * (L * past + L * (L + 1) / 2)
    tf = flops / (ms * 1e-3) / 1e12
    return {"ms": round(ms, 4), "TFLOPs": round(tf, 1), "peak_TFLOPs": 2500.0, "frac": round(tf / 2500.0, 4),
            "tokens_per_s": round(L / (ms * 1e-3), 1), "bound": "mfma",
            "workload": "causal prefill, 4096 new x 32768 prefix, 16q/2kv heads, D=256, bf16 (BASELINE config 2)"}


def bench_prefill_q8(dev, gen, reps=6, warmup=10):
    """The reference's own prefill callable at the same depth: 4096 float32 queries over a 32768-token affine
    8-bit prefix plus the dense chunk (full_attention.py:372 call site)."""
    from moespresso_amd import _lib
    from moespresso_amd.runtime.qwen import kquant

    L, past = 4096, 32768
    q = 0.5 * torch.randn((1, 16, L, 256), device=dev, generator=gen)
    pk = kquant.quantize(0.5 * torch.randn((1, 2, past, 256), device=dev, generator=gen))
    pv = kquant.quantize(0.5 * torch.randn((1, 2, past, 256), device=dev, generator=gen))
    sk = 0.5 * torch.randn((1, 2, L, 256), device=dev, generator=gen)
    sv = 0.5 * torch.randn((1, 2, L, 256), device=dev, generator=gen)
    nbytes = int(_lib.lib().mspr_sdpa_fa_prefill_q8_workspace_bytes(1, 16, 2, L, past))
    ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=dev)
    run = lambda: kquant.sdpa_fa_prefill_q8(q, *pk, *pv, sk, sv, 256 ** -0.5, workspace=ws)
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    # the whole call (conversion of the prefix and of the chunk rows to float16 + the attention kernel), between
    # two events on the launch stream, back to back
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    _lib.profile_enable("flash_prefill")
    e0.record()
    for _ in range(reps):
        run()
    e1.record()
    torch.cuda.synchronize()
    kernel_ms = float(np.mean(_lib.profile_collect("flash_prefill")))
    _lib.profile_enable()
    ms = e0.elapsed_time(e1) / reps
    flops = 4.0 * 256 * 16 * (L * past + L * (L + 1) / 2)
    tf = flops / (ms * 1e-3) / 1e12
    return {"ms": round(ms, 4), "attention_kernel_ms": round(kernel_ms, 4), "TFLOPs": round(tf, 1),
            "frac": round(tf / 2500.0, 4),
            "workload": "sdpa_fa_prefill_q8: 4096 new x 32768-token affine 8-bit prefix, float32 queries; prefix converted to "
                        "bfloat16 rows first, then the bfloat16 MFMA kernel"}


def bench_q8_decode(dev, gen, reps=40):
    """BASELINE config 3: GQA decode over a Q8_0 cache of 37000 tokens, batch 1 and 8."""
    from moespresso_amd import _lib
    from moespresso_amd.runtime.qwen import kquant

    N, out = 37000, {}
    for B in (1, 8):
        sets = []
        for _ in range(4):  # 4 x 322 MB at batch 8: beyond the 256 MB Infinity Cache
            kc = torch.randint(-127, 128, (B, 2, N, 256), device=dev, dtype=torch.int8, generator=gen)
            vc = torch.randint(-127, 128, (B, 2, N, 256), device=dev, dtype=torch.int8, generator=gen)
            ks = (torch.rand((B, 2, N, 8), device=dev, generator=gen) * 0.03).half()
            vs = (torch.rand((B, 2, N, 8), device=dev, generator=gen) * 0.03).half()
            q = torch.randn((B, 16, 256), device=dev, generator=gen).to(torch.bfloat16)
            sets.append((q, kc, ks, vc, vs))
        ws = _lib.q8_decode_workspace(B, 2, N, dev)
        for s_ in sets:
            kquant.sdpa_decode_q8_0(*s_, 256 ** -0.5, workspace=ws)
        torch.cuda.synchronize()
        _lib.profile_enable("q8_decode", "q8_merge")
        for i in range(reps):
            kquant.sdpa_decode_q8_0(*sets[i % 4], 256 ** -0.5, workspace=ws)
        torch.cuda.synchronize()
        split = float(np.mean(_lib.profile_collect("q8_decode"))) * 1e3
        merge = float(np.mean(_lib.profile_collect("q8_merge"))) * 1e3
        _lib.profile_enable()
        nbytes = B * (N * 2 * 2 * (256 + 16) + 16 * 256 * 4)
        out[f"B{B}"] = {"split_us": round(split, 2), "merge_us": round(merge, 2),
                        "GBps": round(nbytes / ((split + merge) * 1e-6) / 1e9, 1),
                        "frac_of_8TBps": round(nbytes / ((split + merge) * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
        del sets
    out["workload"] = "GQA decode, 16q/2kv heads, D=256, 37000-token int8+f16/32 cache (BASELINE config 3)"
    # the reference's own decode callable at the same depth: affine 8-bit cache (group 64, bfloat16 scales and
    # biases as served), float32 queries, batch 1 (runtime/qwen/full_attention.py:323-335 call site)
    sets = []
    for _ in range(4):
        k = kquant.quantize(torch.randn((1, 2, N, 256), device=dev, generator=gen))
        v = kquant.quantize(torch.randn((1, 2, N, 256), device=dev, generator=gen))
        k = (k[0], k[1].to(torch.bfloat16), k[2].to(torch.bfloat16))
        v = (v[0], v[1].to(torch.bfloat16), v[2].to(torch.bfloat16))
        sets.append((torch.randn((1, 16, 1, 256), device=dev, generator=gen), *k, *v))
    ws = _lib.q8_decode_workspace(1, 2, N, dev)
    for s_ in sets:
        kquant.sdpa_decode_q8(*s_, 256 ** -0.5, workspace=ws)
    torch.cuda.synchronize()
    _lib.profile_enable("q8_decode", "q8_merge")
    for i in range(reps):
        kquant.sdpa_decode_q8(*sets[i % 4], 256 ** -0.5, workspace=ws)
    torch.cuda.synchronize()
    split = float(np.mean(_lib.profile_collect("q8_decode"))) * 1e3
    merge = float(np.mean(_lib.profile_collect("q8_merge"))) * 1e3
    _lib.profile_enable()
    nbytes = N * 2 * 2 * (256 + 16) + 16 * 256 * 8
    out["affine_sdpa_decode_q8_B1"] = {
        "split_us": round(split, 2), "merge_us": round(merge, 2),
        "GBps": round(nbytes / ((split + merge) * 1e-6) / 1e9, 1),
        "frac_of_8TBps": round(nbytes / ((split + merge) * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
        "workload": "sdpa_decode_q8: affine 8-bit cache (group 64, bfloat16 scales/biases), float32 queries, "
                    "16q/2kv heads, 37000 keys, batch 1"}
    return out


def bench_ds4_prefill(dev, gen, reps=5):
    """DS4 prefill-side operators at the reference's anchor chunk: 3844 tokens from position 0, 64 heads,
    961 pool rows, top-512, window 128 (wall time per call from torch events on the current stream)."""
    from moespresso_amd import _lib
    from moespresso_amd.runtime.deepseek_v4 import attention_seam_kernel as seam
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak

    T, H, P = 3844, 64, 961

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ts = []
        for _ in range(reps):
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1))
        return round(float(np.median(ts)), 4)

    def kernel_ms(fn):
        """Duration of the consumer kernel alone in the same call (events on the launch stream around the launch;
        the per-call figure above it includes what the host needs to issue the call on an idle device)."""
        _lib.profile_enable("sparse_split")
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        ts = _lib.profile_collect("sparse_split")
        _lib.profile_enable()
        return round(float(np.median(ts)), 4) if ts else None

    q = torch.randn((1, H, T, 512), device=dev, generator=gen).to(torch.float16)
    raw = torch.randn((1, 1, T, 512), device=dev, generator=gen).to(torch.float16)
    comp = torch.randn((1, P, 512), device=dev, generator=gen).to(torch.float16)
    def distinct_sorted_ids(rows):      # 512 distinct pool rows per token, ascending
        keys = torch.rand((T, rows), device=dev, generator=gen)
        return keys.topk(512, dim=1).indices.sort(dim=1).values[None].to(torch.int32).contiguous()

    ids = distinct_sorted_ids(P)
    sinks = torch.randn((H,), device=dev, generator=gen)
    qi = torch.randn((1, H, T, 128), device=dev, generator=gen).to(torch.float16)
    ci = torch.randn((1, P, 128), device=dev, generator=gen).to(torch.float16)
    w = torch.rand((1, T, H), device=dev, generator=gen)
    inv = torch.rand((32,), device=dev, generator=gen)
    out = {
        "indexed_attention_ms": timed(lambda: iak.indexed_mixed_attention_prefill_live_f16(
            q, raw, comp, ids, sinks, pos0=0, window=128, ratio=4)),
        "tiled_scores_ms": timed(lambda: iak.indexer_scores_tiled_live(qi, w, ci, pos0=0, ratio=4)),
        "live_qat_ms": timed(lambda: iak.indexer_q_qat_live(qi.float())),
        "partial_rope_query_ms": timed(lambda: seam.fused_partial_rope(q, inv, offset=0)),
        "workload": "3844-token chunk, 64 heads x 512, 961 pool rows, top-512, window 128 (float16 operands)",
    }
    out["partial_rope_GBps"] = round(2 * q.numel() * 2 / (out["partial_rope_query_ms"] * 1e-3) / 1e9, 1)
    from moespresso_amd.runtime.deepseek_v4 import indexer_score_kernel as isk
    sc = torch.randn((T, P), device=dev, generator=gen)
    out["topk_512_ms"] = timed(lambda: isk.topk_select(sc, 512))
    out["indexed_attention_kernel_ms"] = kernel_ms(lambda: iak.indexed_mixed_attention_prefill_live_f16(
        q, raw, comp, ids, sinks, pos0=0, window=128, ratio=4))
    # the same chunk deep in a context: every token sees its whole window and all 512 selected rows, the pool is
    # larger than one L2 (at position 0 half of the ids lie behind the stop position and their tiles are not run)
    pos_deep = 28000
    p_deep = (pos_deep + T) // 4
    comp_deep = torch.randn((1, p_deep, 512), device=dev, generator=gen).to(torch.float16)
    ids_deep = distinct_sorted_ids(p_deep)
    out["indexed_attention_deep_ms"] = timed(lambda: iak.indexed_mixed_attention_prefill_live_f16(
        q, raw, comp_deep, ids_deep, sinks, pos0=pos_deep, window=128, ratio=4))
    out["indexed_attention_deep_kernel_ms"] = kernel_ms(lambda: iak.indexed_mixed_attention_prefill_live_f16(
        q, raw, comp_deep, ids_deep, sinks, pos0=pos_deep, window=128, ratio=4))
    flop_deep = 4.0 * T * 640 * H * 512
    out["indexed_attention_deep_TFLOPs"] = round(flop_deep / (out["indexed_attention_deep_kernel_ms"] * 1e-3) / 1e12, 1)
    out["indexed_attention_deep_frac_of_2500"] = round(out["indexed_attention_deep_TFLOPs"] / MFMA_PEAK_TFLOPS, 4)
    out["workload_deep"] = f"the same chunk from position {pos_deep}: {p_deep} pool rows, 640 rows per token"
    ci_deep = torch.randn((1, p_deep, 128), device=dev, generator=gen).to(torch.float16)
    out["tiled_scores_deep_ms"] = timed(lambda: iak.indexer_scores_tiled_live(qi, w, ci_deep, pos0=pos_deep, ratio=4))
    sc_deep = torch.randn((T, p_deep), device=dev, generator=gen)
    out["topk_512_deep_ms"] = timed(lambda: isk.topk_select(sc_deep, 512))
    out["tiled_scores_deep_TFLOPs"] = round(2.0 * T * p_deep * H * 128 / (out["tiled_scores_deep_ms"] * 1e-3) / 1e12, 1)
    # the other two forms of the consumer at the same chunk: float32 queries (converted to half into the workspace,
    # then the same kernel) and the banded route (band of 128 positions + every visible pool row at ratio 128)
    q32 = q.float()
    out["indexed_attention_f32_queries_ms"] = timed(lambda: iak.indexed_mixed_attention_prefill_live_f32(
        q32, raw, comp, ids, sinks, pos0=0, window=128, ratio=4))
    out["indexed_attention_f32_queries_deep_ms"] = timed(lambda: iak.indexed_mixed_attention_prefill_live_f32(
        q32, raw, comp_deep, ids_deep, sinks, pos0=pos_deep, window=128, ratio=4))
    p_band = (pos_deep + T) // 128
    comp_band = torch.randn((1, p_band, 512), device=dev, generator=gen).to(torch.float16)
    ids_band = torch.arange(p_band, device=dev, dtype=torch.int32).expand(1, T, p_band).contiguous()
    out["banded_attention_deep_ms"] = timed(lambda: iak.banded_prefill_attention_live(
        q, raw, comp_band, ids_band, sinks, pos0=pos_deep, window=128, ratio=128))
    out["banded_attention_deep_kernel_ms"] = kernel_ms(lambda: iak.banded_prefill_attention_live(
        q, raw, comp_band, ids_band, sinks, pos0=pos_deep, window=128, ratio=128))
    out["workload_banded"] = f"banded route from position {pos_deep}: band 128, {p_band} pool rows at ratio 128, float16 queries"
    return out


def guarded(leg, *args, **kwargs):
    """A side leg of the benchmark: its failure is reported in its place and leaves the headline line intact."""
    try:
        return leg(*args, **kwargs)
    except Exception as exc:  # noqa: BLE001 - whatever a leg raises belongs in the report, not in the exit code
        return {"error": f"{type(exc).__name__}: {exc}"[:300]}


def calibration_copy(dev):
    """One elementwise kernel that reads 1 GiB and writes 1 GiB: the scale of the HBM byte counters."""
    src = torch.ones(1 << 28, device=dev, dtype=torch.float32)
    dst = torch.empty_like(src)
    torch.add(src, 1.0, out=dst)
    torch.cuda.synchronize()
    del src, dst


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--sets", type=int, default=8, help="distinct buffer sets rotated through (cold caches)")
    ap.add_argument("--regions", type=int, default=9, help="timed regions of --steps steps each; the median is reported")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one elementwise kernel that reads 1 GiB and writes 1 GiB (scale for HBM counters)")
    ap.add_argument("--headline-only", action="store_true", help="skip the per-config extras")
    ap.add_argument("--only", default="", help="run just these extras (comma list of prefill, prefill_q8, q8_decode, "
                                               "ds4_prefill) and print them; for counter runs of one kernel")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (every box has one MI355X); rerun with --gpus 1",
              file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        return 2

    from moespresso_amd import _lib
    from moespresso_amd.runtime.deepseek_v4 import indexed_attention_kernel as iak
    from moespresso_amd.runtime.deepseek_v4 import indexer_score_kernel as isk

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(0)
    if args.only:
        legs = {"prefill": bench_prefill, "prefill_q8": bench_prefill_q8, "q8_decode": bench_q8_decode,
                "ds4_prefill": bench_ds4_prefill}
        out = {name: legs[name](dev, gen) for name in args.only.split(",")}
        if args.calibration_copy:
            calibration_copy(dev)
        print(json.dumps(out))
        return 0
    B, R, K, W = args.batch, max(1, args.sets), args.steps, args.warmup
    sets = [make_set(B, dev, gen) for _ in range(R)]
    ws = _lib.sparse_attention_workspace(B, N_HEADS, TOPK + WINDOW, dev)
    scale = K_DIM ** -0.5

    def step(s):
        scores = isk.indexer_scores_fp8(s["qi"], s["keys"], s["kscale"], s["w"])
        sel = isk.topk_select(scores, TOPK)
        return iak.sparse_mla_decode(s["q"], s["kv"], sel, scale=scale, window_start=N_TOKENS - WINDOW,
                                     window_rows=WINDOW, row_mul=4, row_add=3, workspace=ws)

    # eager warm-up (also loads the code objects), then one HIP graph per buffer set
    for s in sets:
        step(s)
    torch.cuda.synchronize()
    graphs, outs = [], []
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for s in sets:
            step(s)
    torch.cuda.current_stream().wait_stream(side)
    for s in sets:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            outs.append(step(s))
        graphs.append(g)
    # A decode step of a model replays the attention of all its layers from one graph: R consecutive layers
    # (the R buffer sets) are also captured as one graph, and the K timed steps are replayed R at a time
    # (the remainder from the per-layer graphs). One graph per layer costs about 5 us more per layer in
    # graph launches.
    layers_graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(layers_graph):
        for s in sets:
            outs.append(step(s))
    torch.cuda.synchronize()

    def replay_steps(n):
        done = 0
        while done + R <= n:
            layers_graph.replay()
            done += R
        while done < n:
            graphs[done % R].replay()
            done += 1

    replay_steps(W)
    torch.cuda.synchronize()
    # a timed region is exactly K steps between two synchronisations; short regions (the driver's K = 20 is about
    # a millisecond) are repeated and the median region is reported
    regions = []
    for _ in range(args.regions):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        replay_steps(K)
        torch.cuda.synchronize()
        regions.append(time.perf_counter() - t0)
    elapsed = float(np.median(regions))
    ms_per_step = elapsed / K * 1e3

    # per-kernel GPU durations: same steps, eager, HIP events around each kernel on its launch stream
    names = ("indexer_fp8", "topk", "sparse_split", "sparse_merge")
    _lib.profile_enable(*names)
    for i in range(K):
        step(sets[i % R])
    torch.cuda.synchronize()
    kernel_us = {n: float(np.mean(_lib.profile_collect(n))) * 1e3 for n in names}
    _lib.profile_enable()

    split_us = kernel_us["sparse_split"]
    achieved = MLA_BYTES_PER_SEQ * B / (split_us * 1e-6) / 1e9
    operator_us = split_us + kernel_us["sparse_merge"]
    roofline = {
        "kernel": "sparse_attn_split_kernel<bf16,576>",
        "bound": "hbm",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        "traffic": measured_traffic_bytes("sparse_attn_split_kernel<2, 576", B * 16) if B == 16 else None,
        "algorithmic_bytes_per_launch": MLA_BYTES_PER_SEQ * B,
        "kernel_us": round(split_us, 2),
        # the same kernel in the committed kernel trace of this benchmark (graph replays, no event records around
        # the launch: events add about 1.5 us); null when the kernel source has changed since the trace was taken
        "kernel_us_traced": traced_kernel_us("sparse_attn_split_kernel<2, 576", f"{B * 16}x1x1"),
        "frac_traced": None,
        # the whole operator (split + merge launches) against the same algorithmic bytes
        "operator_us": round(operator_us, 2),
        "operator_frac": round(MLA_BYTES_PER_SEQ * B / (operator_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
    }
    if roofline["kernel_us_traced"]:
        roofline["frac_traced"] = round(MLA_BYTES_PER_SEQ * B / (roofline["kernel_us_traced"] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)
    # the same kernels at the smaller batches of the configuration (first sequences of the same buffers)
    by_batch = {}
    for bsub in (1, 4):
        if bsub >= B:
            continue
        ws_b = _lib.sparse_attention_workspace(bsub, N_HEADS, TOPK + WINDOW, dev)
        subsets = [{k_: v_[:bsub] for k_, v_ in s_.items()} for s_ in sets]

        def step_b(s_):
            sc = isk.indexer_scores_fp8(s_["qi"], s_["keys"], s_["kscale"], s_["w"])
            se = isk.topk_select(sc, TOPK)
            return iak.sparse_mla_decode(s_["q"], s_["kv"], se, scale=scale, window_start=N_TOKENS - WINDOW,
                                         window_rows=WINDOW, row_mul=4, row_add=3, workspace=ws_b)

        for s_ in subsets:
            step_b(s_)
        torch.cuda.synchronize()
        _lib.profile_enable(*names)
        for i in range(min(K, 64)):
            step_b(subsets[i % R])
        torch.cuda.synchronize()
        by_batch[f"B{bsub}"] = {n_: round(float(np.mean(_lib.profile_collect(n_))) * 1e3, 2) for n_ in names}
        _lib.profile_enable()
    by_batch[f"B{B}"] = {k: round(v, 2) for k, v in kernel_us.items()}
    del sets, graphs, outs
    torch.cuda.empty_cache()

    extras = {
        "kernel_us": {k: round(v, 2) for k, v in kernel_us.items()},
        "kernel_us_by_batch": by_batch,
        "prefill": None if args.headline_only else guarded(bench_prefill, dev, gen),
        "prefill_q8": None if args.headline_only else guarded(bench_prefill_q8, dev, gen),
        "q8_decode": None if args.headline_only else guarded(bench_q8_decode, dev, gen),
        "ds4_prefill": None if args.headline_only else guarded(bench_ds4_prefill, dev, gen),
        "cpu_config1": None if args.no_cpu_baseline else guarded(cpu_config1),
        "cpu_configs_2_3": None if args.no_cpu_baseline else guarded(cpu_other_configs),
        "cpu_baseline_numpy_oracle": None if args.no_cpu_baseline else guarded(cpu_baseline, seconds_budget=6.0),
        "cpu_baseline_1thread": None if args.no_cpu_baseline else guarded(cpu_baseline_torch, seconds_budget=5.0, threads=1),
        "indexer_fp8_GBps": round(IDX_BYTES_PER_SEQ * B / (kernel_us["indexer_fp8"] * 1e-6) / 1e9, 1),
        "tokens_per_s": round(B / (ms_per_step * 1e-3), 1),
        "buffer_sets": R,
        "layers_per_graph_replay": R,
    }
    if args.calibration_copy:
        calibration_copy(dev)

    line = {
        "metric": "sparse decode attn us/layer @128K ctx (indexer score + top-2048 + indexed MLA decode)",
        "value": round(ms_per_step * 1e3, 2),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "timed_regions": args.regions,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"DS4-style sparse decode attention layer, batch {B}: 64x128 indexer over 32768 fp8 keys, "
                        f"top-2048, MLA decode over 2048 gathered + 128 window rows of a 131072-token bf16 cache "
                        f"(576-wide K, 512-wide V, 64 heads)",
            "batch": B,
            "context": N_TOKENS,
        },
        "roofline": roofline,
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline_torch(),
        "extras": extras,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
