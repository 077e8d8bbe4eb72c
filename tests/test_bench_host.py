"""Host-side logic of bench.py, no GPU: the work it prices a launch at, what it does when asked
for more than one GPU, and that the measured-traffic records belong to the device sources in the
tree (a record taken on other sources would be reported as stale and `roofline.traffic` as null)."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402
from flash_distributed_moe_amd import synth  # noqa: E402


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr


def test_algorithmic_work_is_the_closed_form():
    # bytes: active experts x 3*H*I weights + router weights + tokens in and out; flops: T*k*6*H*I + 2*T*H*E
    c2 = synth.CONFIGS["qwen3_30b_decode"]
    assert bench.algorithmic_bytes(c2, 126) == 126 * 3 * 2048 * 768 * 2 + 128 * 2048 * 2 + 2 * 64 * 2048 * 2 == 1190133760
    c3 = synth.CONFIGS["qwen3_30b_prefill"]
    assert bench.algorithmic_flops(c3) == 8192 * 8 * 6 * 2048 * 768 + 2 * 8192 * 2048 * 128 == 622770257920
    c4 = synth.CONFIGS["qwen3_235b_t256"]
    assert bench.algorithmic_bytes(c4, 128) == 128 * 3 * 4096 * 1536 * 2 + 128 * 4096 * 2 + 2 * 256 * 4096 * 2


def test_roofline_bound_of_every_workload():
    assert bench.BOUND["qwen3_30b_prefill"] == "mfma" and bench.BOUND["qwen3_30b_imbalance"] == "mfma"
    assert bench.BOUND.get("qwen3_30b_decode", "hbm") == "hbm" and bench.BOUND.get("qwen3_235b_t256", "hbm") == "hbm"
    assert bench.HBM_PEAK_GBS == 8000.0 and bench.MFMA_BF16_PEAK_TFLOPS == 2500.0


@pytest.mark.parametrize("workload,weights", [("qwen3_30b_decode", "in_place"), ("qwen3_30b_decode", "default"),
                                              ("qwen3_30b_decode", "row_major"), ("qwen3_30b_prefill", "in_place"),
                                              ("qwen3_235b_t256", "in_place"), ("qwen3_235b_t4096", "in_place"),
                                              ("qwen3_30b_imbalance", "in_place")])
def test_traffic_records_belong_to_the_tree(workload, weights):
    traffic, stale = bench.measured_traffic(workload, weights)
    assert traffic is not None, "no measured traffic for this record"
    assert not stale, "profiles/traffic.json was measured on other device sources: re-run the counter passes"
    cfg = synth.CONFIGS[workload]
    # HBM traffic cannot be less than what the launch has to read at least once
    assert traffic >= 0.95 * bench.algorithmic_bytes(cfg, min(cfg.E, 126 if workload == "qwen3_30b_decode" else cfg.E))
