"""bf16-input / fp32-accumulate sgemm (the bf16 variant of benchmark configuration 3).

The reference has no bf16 type, so the oracle is the fp32 result on bf16-rounded inputs
(round to nearest even), as computed by the CPU-generated code of the same program and by
float64 numpy.  Products of two bf16 numbers are exact in fp32, so only the summation order
differs between paths: tolerance max |gpu - ref| <= 2e-2 * max |ref| (the parity statement's
bf16 bound); integer-valued data is exact."""
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")
SMALL = [(128, 192, 128), (48, 40, 24), (200, 150, 100), (1024, 1280, 512)]
RTOL = 2e-2


def to_bf16(a):
    """fp32 -> bf16 bits, round to nearest even (the storage format of p_bfloat16 buffers)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    r = 0x7FFF + ((u >> 16) & 1)
    return ((u + r) >> 16).astype(np.uint16)


def from_bf16(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


def name_of(M, N, K):
    return "sgemm_bf16_%dx%dx%d" % (M, N, K)


def cpu_program(M, N, K):
    n = name_of(M, N, K)
    return runtime.Program(oracle_build.cpu_program_library(PROGRAMS, n), n, needs_gpu_runtime=False)


def test_bf16_rounding_helper():
    # exactly representable values survive; ties go to even
    x = np.array([1.0, -2.5, 0.15625, 3.0e38], np.float32)
    assert np.array_equal(from_bf16(to_bf16(x))[:3], x[:3])
    tie = np.array([0x3F808000], np.uint32).view(np.float32)      # 1.00390625: halfway between two bf16
    assert to_bf16(tie)[0] == 0x3F80
    tie2 = np.array([0x3F818000], np.uint32).view(np.float32)
    assert to_bf16(tie2)[0] == 0x3F82


@pytest.mark.parametrize("M,N,K,what", [(128, 192, 128, "tile 64x64x64, whole tiles"), (48, 40, 24, "tile 64x64x64, guarded edges"),
                                        (200, 150, 100, "tile 64x64x64, guarded edges"), (1024, 1280, 512, "tile 128x128x32, whole tiles"),
                                        (4096, 4096, 4096, "tile 256x256x32, whole tiles")])
def test_every_shape_gets_the_bf16_mfma_kernel(M, N, K, what):
    """Ragged shapes and unaligned rows take the 64x64 tile with guarded loads instead of falling back
    to the schedule-faithful (VALU) kernel."""
    import json
    kernels = json.load(open(os.path.join(PROGRAMS, "build", name_of(M, N, K) + ".o.json")))["kernels"]
    assert len(kernels) == 1 and "v_mfma_f32_32x32x16_bf16" in kernels[0]["how"] and what in kernels[0]["how"]


@pytest.mark.parametrize("M,N,K", SMALL)
def test_cpu_generated_code_matches_float64(M, N, K):
    rng = np.random.RandomState(M + K)
    A, B = to_bf16(rng.uniform(-1, 1, (M, K))), to_bf16(rng.uniform(-1, 1, (K, N)))
    C = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    exact = 1.5 * (from_bf16(A).astype(np.float64) @ from_bf16(B).astype(np.float64)) + 0.5 * C
    cpu_program(M, N, K)(np.array([1.5, 0.5], np.float32), A, B, C)
    assert np.max(np.abs(C - exact)) <= 1e-5 * np.max(np.abs(exact))


def run_gpu(M, N, K, scal, A, B, C):
    from gpu_util import DeviceArray
    d = [DeviceArray(a) for a in (A, B, C)]
    runtime.load(PROGRAMS, name_of(M, N, K))(scal, *[x.buffer() for x in d])
    out = d[2].download()
    for x in d:
        x.free()
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", SMALL)
def test_gpu_matches_cpu_generated_code(M, N, K):
    rng = np.random.RandomState(2 * M + K)
    scal = np.array([1.0, 0.0], np.float32)
    # integer-valued data: exact on every path
    A, B = to_bf16(rng.randint(-5, 5, (M, K)).astype(np.float32)), to_bf16(rng.randint(-5, 5, (K, N)).astype(np.float32))
    C = np.zeros((M, N), np.float32)
    C_cpu = C.copy()
    cpu_program(M, N, K)(scal, A, B, C_cpu)
    assert np.array_equal(run_gpu(M, N, K, scal, A, B, C), C_cpu)
    # uniform data
    A, B = to_bf16(rng.uniform(-1, 1, (M, K))), to_bf16(rng.uniform(-1, 1, (K, N)))
    cpu_program(M, N, K)(scal, A, B, C_cpu)
    out = run_gpu(M, N, K, scal, A, B, C)
    from gpu_util import assert_fp32_parity
    assert_fp32_parity(out, C_cpu, "sgemm bf16 vs CPU-generated code", RTOL)


@pytest.mark.gpu
def test_gpu_4096_sampled_rows():
    M = N = K = 4096
    rng = np.random.RandomState(40)
    scal = np.array([1.0, 0.0], np.float32)
    A, B = to_bf16(rng.uniform(-1, 1, (M, K))), to_bf16(rng.uniform(-1, 1, (K, N)))
    out = run_gpu(M, N, K, scal, A, B, np.zeros((M, N), np.float32))
    rows = rng.choice(M, 32, replace=False)
    exact = from_bf16(A[rows]).astype(np.float64) @ from_bf16(B).astype(np.float64)
    from gpu_util import assert_fp32_parity
    assert_fp32_parity(out[rows], exact, "sgemm bf16 4096^3 sampled rows vs float64", RTOL)
    # integer-valued data: exact
    A, B = to_bf16(rng.randint(-3, 4, (M, K)).astype(np.float32)), to_bf16(rng.randint(-3, 4, (K, N)).astype(np.float32))
    out = run_gpu(M, N, K, scal, A, B, np.zeros((M, N), np.float32))
    exact = from_bf16(A[rows]).astype(np.float64) @ from_bf16(B).astype(np.float64)
    assert np.array_equal(out[rows], exact.astype(np.float32))


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(4096, 3072, 32), (3072, 4096, 160)])
def test_gpu_large_tiles_short_k(M, N, K):
    """256x256 tiles (slices loaded straight into the four-stage LDS ring) with one and five K-slices:
    the ring's start-up, a single steady-state turn and the drain, every element checked, with the
    alpha / beta epilogue."""
    rng = np.random.RandomState(M + K)
    scal = np.array([1.5, 0.5], np.float32)
    A, B = to_bf16(rng.randint(-4, 5, (M, K)).astype(np.float32)), to_bf16(rng.randint(-4, 5, (K, N)).astype(np.float32))
    C = rng.randint(-8, 9, (M, N)).astype(np.float32)
    exact = 1.5 * (from_bf16(A).astype(np.float64) @ from_bf16(B).astype(np.float64)) + 0.5 * C
    assert np.array_equal(run_gpu(M, N, K, scal, A, B, C.copy()), exact.astype(np.float32))     # integer data: exact
    A, B = to_bf16(rng.uniform(-1, 1, (M, K))), to_bf16(rng.uniform(-1, 1, (K, N)))
    exact = 1.5 * (from_bf16(A).astype(np.float64) @ from_bf16(B).astype(np.float64)) + 0.5 * C
    out = run_gpu(M, N, K, scal, A, B, C.copy())
    assert np.max(np.abs(out - exact)) <= 1e-5 * np.max(np.abs(exact))
