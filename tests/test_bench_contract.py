"""What the benchmark driver relies on without a GPU: more than one GPU is refused with a message (every figure
of this build is a single-GPU figure), and the workload names the driver may pass exist."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE)
    assert done.returncode != 0
    assert b"one GPU" in done.stderr + done.stdout


def test_workloads_are_the_benchmark_configurations():
    sys.path.insert(0, ROOT)
    import bench
    assert list(bench.WORKLOADS)[:6] == ["heat2d", "sgemm1024", "sgemm4096", "sgemm4096_bf16", "conv2d", "lstm"]
