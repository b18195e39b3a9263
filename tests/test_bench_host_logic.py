"""Host-side pieces of bench.py that need no GPU: the traffic figure read from the committed counter summary, the
guard around side legs, the one-GPU rule, the algorithmic byte counts."""
import json
import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


COUNTERS = """rocprofv3 HBM traffic counters (test fixture)
source_sha256 sparse_attn.hip {sha}
kernel                                       workgroups  calls    FETCH KiB    WRITE KiB   read MB written MB  total MB
sparse_attn_split_kernel<2, 576, -1, false>         128     24       5308.8       8256.0     10.87       8.45     19.33
sparse_attn_split_kernel<2, 576, -1, false>         256     50      20328.8      16512.0     41.63      16.91     58.54
"""
TRACE = """rocprofv3 kernel trace (test fixture)
source_sha256 sparse_attn.hip {sha}
kernel                                           workgroups threads  calls     avg us  median us     min us
sparse_attn_split_kernel<2, 576, -1, false>         128x1x1     512     72      13.15      13.00      12.48
sparse_attn_split_kernel<2, 576, -1, false>         256x1x1     512   1026      20.14      20.08      19.24
"""


def test_profile_figures_are_read_only_while_the_kernel_source_is_unchanged(tmp_path, monkeypatch):
    counters, trace = tmp_path / "counters.txt", tmp_path / "trace.txt"
    monkeypatch.setattr(bench, "COUNTERS_FILE", str(counters))
    monkeypatch.setattr(bench, "TRACE_FILE", str(trace))
    sha = bench.source_sha256()
    assert sha and len(sha) == 64
    counters.write_text(COUNTERS.format(sha=sha))
    trace.write_text(TRACE.format(sha=sha))
    assert bench.measured_traffic_bytes("sparse_attn_split_kernel<2, 576", 256) == 58540000
    assert bench.measured_traffic_bytes("sparse_attn_split_kernel<2, 576", 12345) is None
    assert bench.measured_traffic_bytes("no_such_kernel", 256) is None
    assert bench.traced_kernel_us("sparse_attn_split_kernel<2, 576", "256x1x1") == 20.14
    assert bench.traced_kernel_us("sparse_attn_split_kernel<2, 576", "128x1x1") == 13.15
    assert bench.traced_kernel_us("sparse_attn_split_kernel<2, 576", "7x1x1") is None
    # a summary taken from another version of the kernel source (or one that does not say) is not quoted
    counters.write_text(COUNTERS.format(sha="0" * 64))
    trace.write_text(TRACE.replace("source_sha256 sparse_attn.hip {sha}\n", ""))
    assert bench.measured_traffic_bytes("sparse_attn_split_kernel<2, 576", 256) is None
    assert bench.traced_kernel_us("sparse_attn_split_kernel<2, 576", "256x1x1") is None


def test_committed_summaries_if_current_agree_with_the_algorithmic_bytes():
    got = bench.measured_traffic_bytes("sparse_attn_split_kernel<2, 576", 256)
    if got is None:      # the kernel source changed after the summary was taken: nothing is quoted
        assert not bench.profile_is_current(bench.COUNTERS_FILE)
        return
    algorithmic = bench.MLA_BYTES_PER_SEQ * 16
    # reads are the algorithmic bytes, the float16 partials of 16 key ranges come on top: between 1.2x and 1.6x
    assert 1.2 * algorithmic < got < 1.6 * algorithmic


def test_algorithmic_bytes_follow_the_configuration():
    # config 5: 2176 rows x 1152 B + q + out + ids; config 4: fp8 keys + scales + q, w + ids
    assert bench.MLA_BYTES_PER_SEQ == 2176 * 1152 + 64 * 576 * 2 + 64 * 512 * 2 + 2048 * 4 == 2654208
    assert bench.IDX_BYTES_PER_SEQ == 32768 * 128 + 32768 * 4 + 64 * 128 * 2 + 64 * 4 + 2048 * 4


def test_a_failing_side_leg_is_reported_in_its_place():
    def leg(x, scale=1):
        return {"value": scale / x}

    assert bench.guarded(leg, 2, scale=4) == {"value": 2.0}
    err = bench.guarded(leg, 0)
    assert set(err) == {"error"} and err["error"].startswith("ZeroDivisionError")
    json.dumps(err)


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode == 2 and "one GPU" in proc.stderr and proc.stdout.strip() == ""
