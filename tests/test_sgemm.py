"""sgemm (benchmark configurations 1 and 3): CPU-generated code vs the numpy restatement, and the MFMA
contraction kernel vs both.

Tolerances (from the parity statement): bit-exact when inputs are small integers (every partial
sum is exactly representable, so summation order cannot matter); for uniform[-1,1] inputs the
MFMA kernel reassociates the k-sum, and the bound is max |gpu - ref| <= 1e-4 * max |ref|, with
ref the CPU-generated code's result (checked in turn against float64)."""
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from oracle import reference_loops as ref
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")
SMALL = [(256, 256, 64), (128, 192, 96), (100, 70, 50), (33, 17, 9), (64, 256, 512)]
RTOL = 1e-4


def name_of(M, N, K):
    return "sgemm_%dx%dx%d" % (M, N, K)


def cpu_program(M, N, K):
    n = name_of(M, N, K)
    return runtime.Program(oracle_build.cpu_program_library(PROGRAMS, n), n, needs_gpu_runtime=False)


def ints(rng, shape):
    return (rng.randint(0, 10, shape) - 5).astype(np.float32)


def uniform(rng, shape):
    return rng.uniform(-1.0, 1.0, shape).astype(np.float32)


@pytest.mark.parametrize("M,N,K", SMALL)
def test_cpu_generated_code_matches_restatement(M, N, K):
    rng = np.random.RandomState(M + N + K)
    A, B, C = ints(rng, (M, K)), ints(rng, (K, N)), ints(rng, (M, N))
    scal = np.array([3.0, 2.0], np.float32)
    expected = ref.sgemm(A, B, C, 3.0, 2.0)
    cpu_program(M, N, K)(scal, A, B, C)
    assert np.array_equal(C, expected)


def test_cpu_generated_code_uniform_inputs_vs_float64():
    M, N, K = 128, 192, 96
    rng = np.random.RandomState(7)
    A, B, C = uniform(rng, (M, K)), uniform(rng, (K, N)), uniform(rng, (M, N))
    exact = 1.0 * (A.astype(np.float64) @ B.astype(np.float64)) + 0.0 * C
    cpu_program(M, N, K)(np.array([1.0, 0.0], np.float32), A, B, C)
    assert np.max(np.abs(C - exact)) <= 1e-5 * np.max(np.abs(exact))


def run_gpu(M, N, K, scal, A, B, C):
    from gpu_util import DeviceArray
    dA, dB, dC = DeviceArray(A), DeviceArray(B), DeviceArray(C)
    runtime.load(PROGRAMS, name_of(M, N, K))(scal, dA.buffer(), dB.buffer(), dC.buffer())
    out = dC.download()
    for d in (dA, dB, dC):
        d.free()
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", SMALL + [(1024, 1024, 1024)])
def test_gpu_integer_inputs_bit_exact(M, N, K):
    rng = np.random.RandomState(3 * M + N)
    A, B, C = ints(rng, (M, K)), ints(rng, (K, N)), ints(rng, (M, N))
    scal = np.array([3.0, 2.0], np.float32)
    C_cpu = C.copy()
    cpu_program(M, N, K)(scal, A, B, C_cpu)
    out = run_gpu(M, N, K, scal, A, B, C)
    assert np.array_equal(out, C_cpu)
    if M * N * K <= 128 * 192 * 96:
        assert np.array_equal(out, ref.sgemm(A, B, C, 3.0, 2.0))


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", SMALL + [(1024, 1024, 1024)])
def test_gpu_uniform_inputs_within_tolerance(M, N, K):
    rng = np.random.RandomState(M + 5 * K)
    A, B, C = uniform(rng, (M, K)), uniform(rng, (K, N)), uniform(rng, (M, N))
    scal = np.array([1.0, 0.0], np.float32)     # the benchmark's alpha and beta
    C_cpu = C.copy()
    cpu_program(M, N, K)(scal, A, B, C_cpu)
    out = run_gpu(M, N, K, scal, A, B, C)
    from gpu_util import assert_fp32_parity
    assert_fp32_parity(out, C_cpu, "sgemm %dx%dx%d vs CPU-generated code" % (M, N, K), RTOL)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,tile", [(2048, 2048, 48, "128x128x16"), (3072, 3072, 32, "192x192x16"),
                                        (1024, 1024, 1024, "64x64x64"), (4096, 4096, 4096, "256x256x16")])
def test_gpu_tile_chosen_for_the_launch(M, N, K, tile):
    """The C tile is the one whose launch is modelled fastest on 256 compute units; the two
    sizes that no other test reaches are also checked for exact results on integer data."""
    text = open(os.path.join(PROGRAMS, "build", name_of(M, N, K) + ".o.hip")).read()
    assert ("tile " + tile + ",") in text
    if K > 64:
        return
    rng = np.random.RandomState(M + K)
    A, B, C = ints(rng, (M, K)), ints(rng, (K, N)), ints(rng, (M, N))
    scal = np.array([3.0, 2.0], np.float32)
    expected = ref.sgemm(A, B, C, 3.0, 2.0)
    assert np.array_equal(run_gpu(M, N, K, scal, A, B, C), expected)


@pytest.mark.gpu
def test_gpu_4096_closed_form_and_sampled_rows():
    M = N = K = 4096
    scal = np.array([1.0, 0.0], np.float32)
    # all ones: C = alpha*K + beta*C exactly (reference: sgemm/cpu/sgemm_wrapper.cpp:166-169)
    ones = np.ones((M, K), np.float32)
    out = run_gpu(M, N, K, np.array([3.0, 2.0], np.float32), ones, ones, np.ones((M, N), np.float32))
    assert np.all(out == np.float32(3.0 * K + 2.0))
    # uniform inputs: sampled rows against float64
    rng = np.random.RandomState(4096)
    A, B = uniform(rng, (M, K)), uniform(rng, (K, N))
    C = np.zeros((M, N), np.float32)
    out = run_gpu(M, N, K, scal, A, B, C)
    rows = rng.choice(M, 48, replace=False)
    exact = A[rows].astype(np.float64) @ B.astype(np.float64)
    from gpu_util import assert_fp32_parity
    assert_fp32_parity(out[rows], exact, "sgemm 4096^3, 48 sampled rows vs float64", RTOL)
    # integer inputs: exact, every row
    A, B = ints(rng, (M, K)), ints(rng, (K, N))
    out = run_gpu(M, N, K, scal, A, B, C)
    exact = (A[rows].astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    assert np.array_equal(out[rows], exact)
    assert np.array_equal(out.sum(axis=1, dtype=np.float64), (A.astype(np.float64) @ B.sum(axis=1, dtype=np.float64)))
