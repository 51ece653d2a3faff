"""conv2d + bias + ReLU (benchmark configuration 4): oracle pins, CPU-generated code vs the oracle, and
the implicit-GEMM MFMA kernel vs both.

Tolerance: bit-exact for integer-valued data; for uniform data max |gpu - ref| <= 1e-4 * max |ref|
(the MFMA kernel sums the 576 products of an output element in a different order)."""
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from oracle import reference_loops as ref
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")
SMALL = [(2, 8, 64, 16), (1, 3, 5, 12), (3, 4, 32, 8)]
RTOL = 1e-4


def name_of(s):
    return "conv2d_%dx%dx%dx%d" % s


def cpu_program(s):
    return runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name_of(s)), name_of(s), needs_gpu_runtime=False)


def make_inputs(s, seed, integer):
    N, CI, CO, H = s
    rng = np.random.RandomState(seed)
    if integer:
        x = rng.randint(0, 6, (N, CI, H, H)).astype(np.float32)
        w = (rng.randint(0, 7, (CO, CI, 3, 3)) - 3).astype(np.float32)
        b = (rng.randint(0, 9, (CO,)) - 4).astype(np.float32)
    else:
        x = rng.uniform(0.0, 1.0, (N, CI, H, H)).astype(np.float32)
        w = rng.uniform(-0.1, 0.1, (CO, CI, 3, 3)).astype(np.float32)
        b = rng.uniform(-0.1, 0.1, (CO,)).astype(np.float32)
    xp = np.zeros((N, CI, H + 2, H + 2), np.float32)
    xp[:, :, 1:-1, 1:-1] = x
    return xp, w, b


def kernel_descriptions(s):
    lib = os.path.join(PROGRAMS, "build", "lib%s.so" % name_of(s))
    return [k["how"] for k in runtime.manifest_of(lib, name_of(s))["kernels"]]


def test_which_kernel_each_shape_gets():
    """The benchmark shape and the small shape with whole tiles take the sliding-window kernel (input staged in LDS
    by channel blocks); the benchmark's 1568 tiles do not divide by the 512 resident workgroups, so its last 32 tiles
    are cut into pieces.  The ragged shapes take the gathering kernel."""
    full, = kernel_descriptions((32, 64, 64, 112))
    assert "sliding window of 9 taps staged in LDS by blocks of 8 channels" in full
    assert "take tiles from a queue, the last tiles cut into 8 pieces" in full
    small, = kernel_descriptions((2, 8, 64, 16))
    assert "sliding window of 9 taps" in small and "cut into" not in small
    for s in [(1, 3, 5, 12), (3, 4, 32, 8)]:
        how, = kernel_descriptions(s)
        assert "gathered operand" in how and "guarded edges" in how


# ---------------------------------------------------------------- oracle pins

def test_oracle_matches_seven_loops():
    xp, w, b = make_inputs((1, 2, 3, 5), 1, integer=True)
    assert np.array_equal(ref.conv2d_bias_relu(xp, w, b), ref.conv2d_bias_relu_loops(xp, w, b))


def test_oracle_special_cases():
    xp, w, b = make_inputs((2, 3, 3, 6), 2, integer=True)
    xp = np.abs(xp)
    # a kernel that is 1 at tap (ky, kx) for co == ci copies the input shifted by (ky-1, kx-1)
    for ky, kx in [(1, 1), (0, 2), (2, 0)]:
        w[:] = 0
        for c in range(3):
            w[c, c, ky, kx] = 1
        out = ref.conv2d_bias_relu(xp, w, np.zeros(3, np.float32))
        assert np.array_equal(out, xp[:, :, ky:ky + 6, kx:kx + 6])
    # centre tap only: a per-pixel matrix product over channels
    w = np.zeros((3, 3, 3, 3), np.float32)
    w[:, :, 1, 1] = np.arange(9, dtype=np.float32).reshape(3, 3)
    out = ref.conv2d_bias_relu(xp, w, np.zeros(3, np.float32))
    assert np.array_equal(out, np.einsum("oc,nchw->nohw", w[:, :, 1, 1], xp[:, :, 1:-1, 1:-1]))
    # ReLU clamps: a large negative bias gives all zeros
    assert np.all(ref.conv2d_bias_relu(xp, w, np.full(3, -1e6, np.float32)) == 0)


@pytest.mark.parametrize("s", SMALL)
def test_cpu_generated_code_matches_oracle(s):
    xp, w, b = make_inputs(s, sum(s), integer=True)
    out = np.zeros((s[0], s[2], s[3], s[3]), np.float32)
    cpu_program(s)(xp, w, b, out)
    assert np.array_equal(out, ref.conv2d_bias_relu(xp, w, b))


# ---------------------------------------------------------------- GPU parity

def run_gpu(s, xp, w, b):
    from gpu_util import DeviceArray
    out = np.zeros((s[0], s[2], s[3], s[3]), np.float32)
    d = [DeviceArray(a) for a in (xp, w, b, out)]
    runtime.load(PROGRAMS, name_of(s))(*[x.buffer() for x in d])
    res = d[3].download()
    for x in d:
        x.free()
    return res


@pytest.mark.gpu
@pytest.mark.parametrize("s", SMALL)
def test_gpu_integer_inputs_bit_exact(s):
    xp, w, b = make_inputs(s, 3 + sum(s), integer=True)
    out_cpu = np.zeros((s[0], s[2], s[3], s[3]), np.float32)
    cpu_program(s)(xp, w, b, out_cpu)
    out = run_gpu(s, xp, w, b)
    assert np.array_equal(out, out_cpu)
    assert np.array_equal(out, ref.conv2d_bias_relu(xp, w, b))


@pytest.mark.gpu
@pytest.mark.parametrize("s", SMALL)
def test_gpu_uniform_inputs_within_tolerance(s):
    xp, w, b = make_inputs(s, 5 + sum(s), integer=False)
    out_cpu = np.zeros((s[0], s[2], s[3], s[3]), np.float32)
    cpu_program(s)(xp, w, b, out_cpu)
    out = run_gpu(s, xp, w, b)
    from gpu_util import assert_fp32_parity
    assert_fp32_parity(out, out_cpu, "conv2d vs CPU-generated code", RTOL)


@pytest.mark.gpu
def test_gpu_full_size():
    s = (32, 64, 64, 112)
    # integer-valued data: exact against the float64 restatement
    xp, w, b = make_inputs(s, 112, integer=True)
    assert np.array_equal(run_gpu(s, xp, w, b), ref.conv2d_bias_relu(xp, w, b))
    # the benchmark's distributions: within tolerance of the float64 restatement
    xp, w, b = make_inputs(s, 113, integer=False)
    out, exact = run_gpu(s, xp, w, b), ref.conv2d_bias_relu(xp, w, b)
    from gpu_util import assert_fp32_parity
    assert_fp32_parity(out, exact, "conv2d vs float64 restatement", RTOL)
    # linearity in the input away from the clamp: conv(2x) - 2 conv(x) + bias term
    assert np.count_nonzero(out) > 0.3 * out.size
