"""Sums whose reduction loop is mapped to GPU threads (tests/programs/thread_reductions.cpp): the HIP
back-end lowers them to private partial sums, DPP reductions across the lanes of a wavefront (through
LDS across wavefronts) and one update of the element.  Checked against numpy: bit-exact on
integer-valued data (any summation order gives the same fp32 result while the sums stay below 2^24),
within 1e-4 relative (element by element, with a stated absolute allowance) on uniform data, whose
sums the GPU forms in another order than the serial CPU loop."""
import os
import re

import numpy as np
import pytest

from oracle import build as oracle_build
from tiramisu_amd import runtime

CASES = {
    # name: (rows, columns, initial value, takes a vector)
    "gemv_wavefront": (300, 1000, 0.0, True),
    "row_sums_quarter_wave": (128, 50, 1.0, False),
    "row_sums_block": (40, 5000, 0.0, False),
}


def inputs(name, integer, seed):
    M, N, init, vec = CASES[name]
    rng = np.random.RandomState(seed)
    draw = (lambda shape: (rng.randint(0, 10, shape) - 5).astype(np.float32)) if integer else \
        (lambda shape: rng.uniform(-1, 1, shape).astype(np.float32))
    A = draw((M, N))
    x = draw((N,)) if vec else None
    expected = init + (A.astype(np.float64) @ x.astype(np.float64) if vec else A.astype(np.float64).sum(axis=1))
    return A, x, expected


def call(prog, A, x, out):
    if x is None:
        prog(A, out)
    else:
        prog(A, x, out)


@pytest.mark.parametrize("name", sorted(CASES))
def test_lowered_to_wavefront_reductions(programs_dir, name):
    text = open(os.path.join(programs_dir, "build", name + ".o.hip")).read()
    how = re.search(r"^// _kernel_\d+: (.*)$", text, re.M).group(1)
    assert "DPP wavefront reductions" in how
    assert ("through LDS" in how) == (name == "row_sums_block")
    assert "twave::" in text and "_partial0" in text


@pytest.mark.parametrize("name", sorted(CASES))
def test_cpu_generated_code_matches_numpy(programs_dir, name):
    A, x, expected = inputs(name, True, 1)
    out = np.full((A.shape[0],), -7.0, np.float32)
    cpu = runtime.Program(oracle_build.cpu_program_library(programs_dir, name), name, needs_gpu_runtime=False)
    call(cpu, A, x, out)
    assert np.array_equal(out, expected.astype(np.float32))


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_gpu_matches_numpy(programs_dir, name):
    from gpu_util import DeviceArray, assert_fp32_parity
    prog = runtime.load(programs_dir, name)
    for integer in (True, False):
        A, x, expected = inputs(name, integer, 2 + integer)
        out = np.full((A.shape[0],), -7.0, np.float32)
        dev = [DeviceArray(a) for a in ([A, out] if x is None else [A, x, out])]
        print("running", name, "integer" if integer else "uniform", flush=True)
        prog(*[d.buffer() for d in dev])
        got = dev[-1].download()
        for d in dev:
            d.free()
        if integer:
            assert np.array_equal(got, expected.astype(np.float32))
        else:
            assert_fp32_parity(got, expected, name + " vs float64 numpy", 1e-4)


def test_sum_across_wavefronts_under_a_condition_keeps_the_barrier_out(programs_dir):
    """tests/programs/thread_reduction_under_condition.cpp: the 256-thread loop sits under `if (block iterator >= 3)`.
    The lowering across wavefronts ends in a workgroup barrier that every thread must reach, so the emitter must not
    use it below a condition: the loop stays as the program states it (no LDS stage, no barrier below the condition)."""
    text = open(os.path.join(programs_dir, "build", "row_sums_from_row_3.o.hip")).read()
    kernel = text[text.index('extern "C" __global__'):]
    assert "if ((c1 >= 3))" in kernel
    # (the initialisation above the condition, which no thread loop encloses, runs on the first thread between barriers)
    assert "block_group_sum" not in kernel and "__syncthreads" not in kernel[kernel.index("if ((c1 >= 3))"):]
    assert "DPP wavefront reductions" not in re.search(r"^// _kernel_\d+: (.*)$", text, re.M).group(1)
