"""Host-side pieces of bench.py that need no GPU: the traffic figure read from the committed counter summary, the
guard around side legs, the one-GPU rule, the algorithmic byte counts."""
import json
import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_traffic_comes_from_the_committed_counter_summary():
    got = bench.measured_traffic_bytes("sparse_attn_split_kernel<2, 576", 256)
    algorithmic = bench.MLA_BYTES_PER_SEQ * 16
    # reads are the algorithmic bytes, the float16 partials of 16 key ranges come on top: between 1.2x and 1.6x
    assert got is not None and 1.2 * algorithmic < got < 1.6 * algorithmic
    assert bench.measured_traffic_bytes("sparse_attn_split_kernel<2, 576", 12345) is None
    assert bench.measured_traffic_bytes("no_such_kernel", 256) is None


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
