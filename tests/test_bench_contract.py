"""bench.py's side of the driver contract that can be checked without a GPU: the refusal of more than one GPU, the
algorithmic-byte formulas behind `value` and `roofline.achieved` against the per-row and per-token byte counts
(hand-expanded at the headline shape), and that every traffic constant names a committed profile."""
import importlib.util
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert res.returncode != 0
    assert "one GPU" in (res.stderr + res.stdout)


def test_algorithmic_bytes_at_the_headline_shape():
    b = _bench()
    T, H, K, E, R = 8192, 7168, 8, 256, 8
    N_r, N_e = 43456, 65536                     # what the benchmark's seed routes (uniform top-8 of 256)
    ab = b.algorithmic_bytes(T, H, K, E, R, N_r, N_e, fp8=True, expanded=False)
    # dispatch: every token read once (2H), its indices and weights read (K * 12), and per received row the FP8 payload,
    # one fp32 scale per 128 channels, the row's indices (int64), weights (fp32) and K + 2 metadata words
    row = H + 4 * (H // 128) + K * 8 + K * 4 + (K + 2) * 4
    assert ab["dispatch"] == T * 2 * H + T * K * 12 + N_r * row == 445363712
    # combine: every received row read as BF16, the routing read, every token written as BF16
    assert ab["combine"] == N_r * 2 * H + T * K * 8 + T * 2 * H == 740950016
    assert ab["layout"] == T * K * 8 + T * R + (R + E) * 4 == 590880
    exp = b.algorithmic_bytes(T, H, K, E, R, N_r, N_e, fp8=True, expanded=True)
    assert exp["dispatch"] == T * 2 * H + T * K * 12 + N_e * (H + 4 * (H // 128) + 4) + N_r * (K + 2) * 4
    assert exp["combine"] == N_e * 2 * H + T * K * 8 + T * 2 * H
    bf16 = b.algorithmic_bytes(T, H, K, E, R, N_r, N_e, fp8=False, expanded=False)
    assert bf16["dispatch"] == T * 2 * H + T * K * 12 + N_r * (2 * H + K * 8 + K * 4 + (K + 2) * 4)


def test_traffic_constants_point_at_committed_profiles():
    b = _bench()
    assert b.HBM_PEAK_GBS == 8000.0
    text = open(os.path.join(ROOT, "bench.py")).read()
    for name in ("bench_C3_hbm_counters.md", "bench_C4_C2_hbm_counters.md", "bench_C5_low_latency_hbm_counters.md"):
        assert name in text and os.path.exists(os.path.join(ROOT, "profiles", name)), name
    for key, value in b.MEASURED_TRAFFIC_BYTES.items():
        assert isinstance(value, int) and value > 0, key
    # measured traffic is close to, and not below, the algorithmic bytes of the same call
    ab = b.algorithmic_bytes(8192, 7168, 8, 256, 8, 43456, 65536)
    measured = b.MEASURED_TRAFFIC_BYTES[("C3", "compact", "fp8", "combine")]
    assert 1.0 <= measured / ab["combine"] < 1.05


@pytest.mark.gpu
def test_wave_spans_through_the_measurement_build():
    """`bench.py --wave-spans` (the command of profiles/dispatch_wave_spans_C3.md): the measurement build runs the same
    dispatch, and what it records is consistent - every mover wavefront stamped, the span of the wavefronts inside the
    launch-to-launch time, the single launch's head later than that of a move on a finished layout."""
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--no-cpu-baseline", "--wave-spans", "--steps", "3",
                          "--warmup", "2"], capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, res.stderr[-2000:]
    line = json.loads(res.stdout.strip().splitlines()[-1])
    spans = line["wave_spans_us"]
    assert spans["wavefronts"] == 8192 * 4
    for name in ("dispatch", "dispatch_move"):
        s = spans[name]
        assert 0 < s["first_wavefront_done"] < s["last_wavefront_start"] < s["first_start_to_last_store_acknowledged"]
        assert s["first_start_to_last_store_issued"] <= s["first_start_to_last_store_acknowledged"] < s["launch_to_launch"] + 10
        assert 1 < s["median_wavefront_lifetime"] < 60
    assert spans["dispatch"]["first_wavefront_done"] > spans["dispatch_move"]["first_wavefront_done"]
