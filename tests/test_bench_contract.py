"""bench.py's `roofline.traffic` comes from the committed rocprofv3 counter summary, not from constants
in the script: the summary parses, and what it yields is consistent with the workloads' algorithmic bytes."""

import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_traffic_is_read_from_the_committed_counter_summary():
    import bench

    assert os.path.exists(bench.TRAFFIC_PROFILE)
    c2, c4 = bench.measured_traffic("c2"), bench.measured_traffic("c4")
    assert c2 is not None and c4 is not None
    # prefill c2 moves at least its inputs and outputs (factors 47.2 MB in, O + LSE 68.2 MB out); its step
    # writes dense Q, K, V (201.3 MB) and reads them back at least once on top of that
    _, B, lq, lk, H, D, rq, rk, _ = bench.WORKLOADS["c2"]
    algorithmic = (B * lq * rq * (H + D) + 2 * B * lk * rk * (H + D) + B * lq * H * D) * 2 + B * H * lq * 4
    dense = 3 * B * lq * H * D * 2
    assert algorithmic + 2 * dense <= c2 <= algorithmic + 4 * dense
    # decode c4 reads its cache once: within 5 % of the algorithmic bytes
    _, B, lq, lk, H, D, rq, rk, _ = bench.WORKLOADS["c4"]
    assert 1.0 <= c4 / bench.decode_bytes(B, lq, lk, H, D, rq, rk) <= 1.05
    # a workload without a counter run reports none
    assert bench.measured_traffic("c5") is None


def test_more_than_one_gpu_is_refused_with_a_message():
    """Nothing in this build uses a second GPU: `--gpus N` with N above 1 exits and says so, before any device is touched."""
    import subprocess

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)


def test_every_workload_has_a_known_kind_and_the_default_is_the_headline_configuration():
    import bench

    assert bench.WORKLOADS["c2"] == ("prefill", 4, 4096, 4096, 16, 128, 6, 2, True)
    assert bench.WORKLOADS["c4"][:8] == ("decode", 64, 1, 8192, 32, 128, 6, 2)
    assert {w[0] for w in bench.WORKLOADS.values()} <= {"prefill", "decode", "dense", "append", "backward"}
    # the published peaks the rooflines are priced against
    assert (bench.PEAK_BF16_TFLOPS, bench.PEAK_F32_TFLOPS, bench.PEAK_HBM_GBS) == (2516.6, 157.3, 8000.0)
