"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py): seeded inputs
with the outputs the pinned oracle gave.  The oracle, the CPU-generated code and the HIP kernels
are all compared with those bytes."""
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from oracle import reference_loops as ref
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")
BENCH_PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")
TEST_PROGRAMS = os.path.join(ROOT, "tests", "programs")
LSTM_TOL = 1e-6   # the oracle's matrix products go through the host BLAS, whose summation order may differ


def fixture(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False)


def cases():
    """name -> (programs dir, function, inputs in argument order, index of the output, expected, tolerance)"""
    s = fixture("sgemm_33x17x9")
    h = fixture("heat2d_20x2")
    c = fixture("conv2d_1x3x5x12")
    l = fixture("lstm_1x4x16x3")
    r = fixture("resample_bilinear_90x132")
    planes = np.zeros((2, 20, 20), np.float32)
    planes[0] = h["grid"]
    return {
        "sgemm": (BENCH_PROGRAMS, "sgemm_33x17x9", [("host", np.array([s["alpha"], s["beta"]], np.float32)), s["A"], s["B"], s["C"].copy()],
                  3, s["out"], 0.0),
        "heat2d": (BENCH_PROGRAMS, "heat2d_20x2", [planes], 0, h["planes"], 0.0),
        "conv2d": (BENCH_PROGRAMS, "conv2d_1x3x5x12", [c["x"], c["w"], c["b"], np.zeros_like(c["out"])], 3, c["out"], 0.0),
        "lstm": (BENCH_PROGRAMS, "lstm_1x4x16x3", [l["w"], l["b"], l["x"], np.zeros_like(l["y"])], 3, l["y"], 1e-4),
        "resample": (TEST_PROGRAMS, "resample_bilinear", [r["src"], np.zeros_like(r["out"])], 1, r["out"], 0.0),
    }


def close(got, want, tol):
    if tol == 0.0:
        return np.array_equal(got, want)
    return np.max(np.abs(got - want)) <= tol * max(1.0, float(np.max(np.abs(want))))


def test_oracle_reproduces_the_fixtures():
    s = fixture("sgemm_33x17x9")
    assert np.array_equal(ref.sgemm(s["A"], s["B"], s["C"], float(s["alpha"]), float(s["beta"])), s["out"])
    h = fixture("heat2d_20x2")
    assert np.array_equal(ref.heat2d(h["grid"], 2), h["planes"])
    c = fixture("conv2d_1x3x5x12")
    assert np.array_equal(ref.conv2d_bias_relu(c["x"], c["w"], c["b"]), c["out"])
    l = fixture("lstm_1x4x16x3")
    assert close(ref.lstm(l["w"], l["b"], l["x"]), l["y"], LSTM_TOL)
    r = fixture("resample_bilinear_90x132")
    assert np.array_equal(ref.resample_bilinear(r["src"]), r["out"])


@pytest.mark.parametrize("name", ["sgemm", "heat2d", "conv2d", "lstm", "resample"])
def test_cpu_generated_code_reproduces_the_fixtures(name):
    directory, fn, inputs, out_index, expected, tol = cases()[name]
    args = [a[1] if isinstance(a, tuple) else a for a in inputs]
    runtime.Program(oracle_build.cpu_program_library(directory, fn), fn, needs_gpu_runtime=False)(*args)
    assert close(args[out_index], expected, tol)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["sgemm", "heat2d", "conv2d", "lstm", "resample"])
def test_gpu_reproduces_the_fixtures(name):
    from gpu_util import DeviceArray
    directory, fn, inputs, out_index, expected, tol = cases()[name]
    devs, args = {}, []
    for i, a in enumerate(inputs):
        if isinstance(a, tuple):
            args.append(a[1])
        else:
            devs[i] = DeviceArray(a)
            args.append(devs[i].buffer())
    runtime.load(directory, fn)(*args)
    assert close(devs[out_index].download(), expected, tol)
