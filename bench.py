#!/usr/bin/env python3
"""Benchmark of the Tiramisu HIP back-end on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|heat2d|sgemm1024|sgemm4096|...]

Prints ONE JSON line.  The headline is BASELINE config 2 (heat2d 8192x8192, 32 time steps,
the configuration the HBM-roofline target is quoted on): `value` is algorithmic HBM GB/s of the
whole compiled Tiramisu function with its buffers already resident in HBM.  A "step" is one
call of the compiled function (32 stencil time steps).  The other configurations that exist
as compiled programs are measured the same way and reported under "workloads".

`roofline` is measured per kernel with HIP events around every launch (the runtime ABI's
tiramisu_hip_profile_*), on the stream the generated code launches on.  `cpu_baseline` times
the CPU-generated code of the same Tiramisu program (the oracle's CPU back-end restatement:
parallelize + vectorize schedule, OpenMP) on the host cores of this machine.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix
BF16_MFMA_PEAK_TFLOPS = 2500.0
PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")

# HBM bytes per launch of the dominant heat2d kernel measured with rocprofv3 --pmc
# (FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of known size); see profiles/.
HEAT2D_TRAFFIC_BYTES_PER_LAUNCH = {5: (165113.3 * 2.000 + 262080.0 * 1.000) * 1024}  # by time steps per launch


def device_array(host):
    from gpu_util import DeviceArray
    return DeviceArray(host)


def time_steps(call, steps, warmup):
    from tiramisu_amd import runtime
    w = runtime.wrappers()
    for _ in range(warmup):
        call()
    w.tiramisu_hip_stream_synchronize(0)
    t0 = time.perf_counter()
    for _ in range(steps):
        call()
    w.tiramisu_hip_stream_synchronize(0)
    return (time.perf_counter() - t0) * 1e3 / steps


def kernel_profile(call, steps):
    """Average duration per kernel name over `steps` calls, HIP events around every launch."""
    from tiramisu_amd import runtime
    recs = runtime.profile(lambda: [call() for _ in range(steps)])
    by = {}
    for name, ms in recs:
        by.setdefault(name, []).append(ms)
    return {k: (float(np.mean(v)), len(v) // steps) for k, v in by.items()}


def cpu_time(call, min_seconds=3.0, max_runs=5):
    call()  # warm-up
    ts = []
    t_all = time.perf_counter()
    while len(ts) < max_runs and (len(ts) < 1 or time.perf_counter() - t_all < min_seconds):
        t0 = time.perf_counter()
        call()
        ts.append(time.perf_counter() - t0)
    return float(np.median(ts)), len(ts)


def cpu_threads():
    return int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))


# ---------------------------------------------------------------- workloads

def bench_heat2d(steps, warmup, with_cpu):
    from tiramisu_amd import runtime
    from oracle import build as oracle_build
    n, tsteps = 8192, 32
    name = "heat2d_%dx%d" % (n, tsteps)
    rng = np.random.RandomState(2)
    planes = np.zeros((2, n, n), np.float32)
    planes[0, 1:-1, 1:-1] = rng.uniform(0.0, 1.0, (n - 2, n - 2)).astype(np.float32)
    dev = device_array(planes)
    prog = runtime.load(PROGRAMS, name)
    buf = dev.buffer()
    ms = time_steps(lambda: prog(buf), steps, warmup)
    alg_bytes = tsteps * 2.0 * n * n * 4
    prof = kernel_profile(lambda: prog(buf), steps)
    # dominant kernel: the one with the largest total time per call
    dom = max(prof.items(), key=lambda kv: kv[1][0] * kv[1][1])
    fused_steps = int(round((tsteps - 2) / dom[1][1])) if dom[1][1] else 1
    per_launch_bytes = fused_steps * 2.0 * n * n * 4
    achieved = per_launch_bytes / (dom[1][0] * 1e-3) / 1e9
    out = {
        "value": alg_bytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": ms,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": HEAT2D_TRAFFIC_BYTES_PER_LAUNCH.get(fused_steps),
                     "kernel": dom[0], "kernel_ms": dom[1][0], "launches_per_step": dom[1][1],
                     "time_steps_per_launch": fused_steps},
        "kernels": {k: {"ms": v[0], "launches_per_step": v[1]} for k, v in prof.items()},
    }
    if with_cpu:
        cpu = runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)
        host = planes.copy()
        sec, runs = cpu_time(lambda: cpu(host))
        out["cpu_baseline"] = {"value": alg_bytes / sec / 1e9, "unit": "GB/s", "cores": cpu_threads(), "kind": "port",
                               "sample": "whole workload (8192x8192, 32 steps), median of %d runs of the CPU-generated "
                                         "code (parallelize y, vectorize x by 8; g++ -O2 -mavx, OpenMP)" % runs}
    dev.free()
    return out


def bench_sgemm(M, steps, warmup, with_cpu):
    from tiramisu_amd import runtime
    from oracle import build as oracle_build
    N = K = M
    name = "sgemm_%dx%dx%d" % (M, N, K)
    rng = np.random.RandomState(M)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    C = np.zeros((M, N), np.float32)
    scal = np.array([1.0, 0.0], np.float32)
    dA, dB, dC = device_array(A), device_array(B), device_array(C)
    prog = runtime.load(PROGRAMS, name)
    args = (scal, dA.buffer(), dB.buffer(), dC.buffer())
    ms = time_steps(lambda: prog(*args), steps, warmup)
    flop = 2.0 * M * N * K
    prof = kernel_profile(lambda: prog(*args), steps)
    dom = max(prof.items(), key=lambda kv: kv[1][0] * kv[1][1])
    achieved = flop / (dom[1][0] * 1e-3) / 1e12
    out = {
        "value": flop / (ms * 1e-3) / 1e9, "unit": "GFLOP/s", "ms_per_step": ms,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / FP32_MFMA_PEAK_TFLOPS, "traffic": None, "kernel": dom[0], "kernel_ms": dom[1][0]},
    }
    if with_cpu:
        cpu = runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)
        Ch = C.copy()
        sec, runs = cpu_time(lambda: cpu(scal, A, B, Ch), min_seconds=2.0, max_runs=3)
        out["cpu_baseline"] = {"value": flop / sec / 1e9, "unit": "GFLOP/s", "cores": cpu_threads(), "kind": "port",
                               "sample": "whole workload (%d^3), median of %d runs of the CPU-generated code "
                                         "(parallelize i, vectorize j by 8)" % (M, runs)}
    for d in (dA, dB, dC):
        d.free()
    return out


def bench_copy(steps, warmup, with_cpu):
    """Plain 256 MiB -> 256 MiB copy (schedule-faithful kernel): counter calibration."""
    from tiramisu_amd import runtime
    n = 8192
    a = np.ones((n, n), np.float32)
    dS, dD = device_array(a), device_array(a)
    prog = runtime.load(PROGRAMS, "copy_plane")
    args = (dS.buffer(), dD.buffer())
    ms = time_steps(lambda: prog(*args), steps, warmup)
    nbytes = 2.0 * n * n * 4
    out = {"value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": ms,
           "roofline": {"bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": nbytes}}
    dS.free()
    dD.free()
    return out


WORKLOADS = {
    "heat2d": lambda s, w, c: bench_heat2d(s, w, c),
    "sgemm1024": lambda s, w, c: bench_sgemm(1024, s, w, c),
    "sgemm4096": lambda s, w, c: bench_sgemm(4096, s, w, c),
}
try:
    import bench_more  # noqa: F401  (further workloads register themselves when present)
except ImportError:
    pass


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: this back-end compiles single-GPU Tiramisu programs and nothing here "
                 "uses a second device (run with --gpus 1)")
    from tiramisu_amd import runtime
    if runtime.wrappers().tiramisu_hip_device_count() < 1:
        sys.exit("no HIP device visible")
    WORKLOADS["copy"] = bench_copy   # calibration only, not part of "all"
    names = [n for n in WORKLOADS if n != "copy"] if a.workload == "all" else [a.workload]
    results = {}
    for n in names:
        with_cpu = (not a.no_cpu) and (a.workload != "all" or n in ("heat2d", "sgemm1024"))
        results[n] = WORKLOADS[n](a.steps, a.warmup, with_cpu)
    head_name = "heat2d" if "heat2d" in results else names[0]
    head = results[head_name]
    line = {
        "metric": "GFLOP/s (sgemm, conv2d, LSTM) + HBM GB/s (heat2d), % of roofline, 1 GPU",
        "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (seeded uniform inputs, already resident in HBM)",
        "config": {"workload": {"heat2d": "heat2d 5-point stencil, fp32 grid 8192x8192, 32 time steps (BASELINE configs[1])",
                                "sgemm1024": "sgemm fp32 1024^3 (BASELINE configs[0])",
                                "sgemm4096": "sgemm fp32 4096^3 (BASELINE configs[2])"}.get(head_name, head_name)},
        "roofline": head["roofline"],
        "cpu_baseline": head.get("cpu_baseline"),
        "workloads": {k: v for k, v in results.items() if k != head_name},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
