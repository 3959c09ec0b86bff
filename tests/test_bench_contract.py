"""bench.py's contract where it can be checked without a GPU: one GPU only, no CPU fallback, and the figures it
quotes from the committed rocprofv3 summaries are there and say what the line claims."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

N = 16 << 20


def run_bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    p = run_bench("--gpus", "2")
    assert p.returncode != 0
    assert "--gpus must be 1" in p.stderr and "one GPU" in p.stderr
    assert p.stdout.strip() == ""                        # no JSON line that could pass for a measurement


def test_no_gpu_means_no_number():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    p = run_bench("--steps", "2", "--warmup", "1")
    assert p.returncode != 0
    assert "no CPU fallback" in p.stderr
    assert p.stdout.strip() == ""


def test_profile_figures_the_line_quotes():
    import bench
    avg = bench.avg_from_profile("k_merged")
    traffic = bench.traffic_from_profile("k_merged")
    assert avg is not None and traffic is not None, "profiles/ lacks the KERNEL_AVG / TRAFFIC line of the headline kernel"
    # the headline kernel: 5N algorithmic bytes in 10-16 us, and no more than 4.1N across the fabric (the sum blocks'
    # read of the local tensor must stay an L2 hit; a change of block placement would show here)
    assert 10.0 < avg < 16.0
    assert 3.9 * N < traffic <= 4.1 * N
    for k in ("k_step_sum", "k_step_pack"):
        assert bench.avg_from_profile(k) and bench.traffic_from_profile(k)
    assert abs(bench.traffic_from_profile("k_step_sum") / N - 3.0) < 0.05
    assert abs(bench.traffic_from_profile("k_step_pack") / N - 2.0) < 0.05
    assert bench.avg_from_profile("no_such_kernel") is None


def test_own_warmup_covers_the_rotation():
    import bench
    assert bench.own_warmup(5, 16, 12) >= 2 * 48          # two periods of 16 slots x 12 tensors
    assert bench.own_warmup(500, 16, 12) == 500
    assert bench.own_warmup(0, 4, 1) >= 48
