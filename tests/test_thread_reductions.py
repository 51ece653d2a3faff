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
    "row_sums_ragged_rows_block": (10, 558, 1.0, False),
    "row_sums_100_lanes": (31, 450, 1.0, False),
    "row_sums_26_of_64_lanes": (80, 26, 0.0, False),
    "row_sums_int32_wave": (50, 45, 1, False),
    "row_sums_int32_block": (33, 700, 1, False),
    "row_sums_float64_wave": (37, 333, 1.0, False),
    "row_sums_int64_block": (21, 900, 1, False),
    "row_sums_uint8_wave": (45, 700, 0, False),
    "row_sums_int16_block": (19, 1300, 1, False),
    "row_maxima_wave": (41, 500, None, False),
    "row_minima_int32_block": (10, 900, None, False),
    "row_maxima_int8_wave": (30, 333, None, False),
}
EXTREMES = {"row_maxima_wave": (np.float32, np.max), "row_minima_int32_block": (np.int32, np.min), "row_maxima_int8_wave": (np.int8, np.max)}
ACROSS_WAVEFRONTS = {"row_sums_block", "row_sums_ragged_rows_block", "row_sums_100_lanes", "row_sums_int32_block", "row_sums_int64_block", "row_sums_int16_block", "row_minima_int32_block"}
INT32 = {"row_sums_int32_wave", "row_sums_int32_block", "row_sums_float64_wave", "row_sums_int64_block", "row_sums_uint8_wave", "row_sums_int16_block", "row_maxima_wave", "row_minima_int32_block", "row_maxima_int8_wave"}       # exact sums only


def inputs(name, integer, seed):
    M, N, init, vec = CASES[name]
    rng = np.random.RandomState(seed)
    draw = (lambda shape: (rng.randint(0, 10, shape) - 5).astype(np.float32)) if integer else \
        (lambda shape: rng.uniform(-1, 1, shape).astype(np.float32))
    if name in EXTREMES:
        dtype, pick = EXTREMES[name]
        A = rng.uniform(-1000, 1000, (M, N)).astype(dtype) if dtype == np.float32 else rng.randint(np.iinfo(dtype).min, np.iinfo(dtype).max + 1, (M, N)).astype(dtype)
        return A, None, pick(A, axis=1)
    if name in INT32:
        if name == "row_sums_uint8_wave":
            A = rng.randint(0, 256, (M, N)).astype(np.uint8)
            return A, None, ((init + A.sum(axis=1, dtype=np.int64)) % 256)
        if name == "row_sums_int16_block":
            A = rng.randint(-2 ** 15, 2 ** 15, (M, N)).astype(np.int16)
            return A, None, (init + A.sum(axis=1, dtype=np.int64)).astype(np.int16)          # wraps
        if name == "row_sums_int64_block":
            A = rng.randint(-2 ** 50, 2 ** 50, (M, N)).astype(np.int64)
        elif name == "row_sums_float64_wave":
            A = rng.randint(-2 ** 40, 2 ** 40, (M, N)).astype(np.float64)         # beyond fp32's 24 bits, exact in fp64
        else:
            A = rng.randint(-2 ** 20, 2 ** 20, (M, N)).astype(np.int32)
        return A, None, init + A.sum(axis=1, dtype=np.float64 if A.dtype == np.float64 else np.int64)
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
    assert ("through LDS" in how) == (name in ACROSS_WAVEFRONTS)
    assert "twave::" in text and "_partial0" in text


def test_rows_beyond_the_last_tile_carry_a_predicate_and_reach_the_barrier(programs_dir):
    """Four rows of 256 threads per workgroup, 10 rows: the row loop's guard must not enclose the sum across
    wavefronts (its barrier is for every thread); the statements run under a predicate instead."""
    text = open(os.path.join(programs_dir, "build", "row_sums_ragged_rows_block.o.hip")).read()
    kernel = text[text.index('extern "C" __global__'):]
    assert "const bool _live_c3 = " in kernel
    at = kernel.index("block_group_sum<256>")
    before = kernel[:at]
    assert before.count("{") - before.count("}") == 4        # kernel, block loop, row loop, the sum's own scope: no `if` open
    assert "if (threadIdx.x == 255 && _live_c3)" in kernel


def test_a_width_between_the_supported_ones_is_rounded_up(programs_dir):
    for name, width, last in (("row_sums_100_lanes", "block_group_sum<128>", 99), ("row_sums_26_of_64_lanes", "wave_group_sum<32>", 25)):
        text = open(os.path.join(programs_dir, "build", name + ".o.hip")).read()
        assert width in text
        assert re.search(r"c5 >= 0 && c5 <= %d\)" % last, text), name       # the lanes beyond the loop's extent add nothing
        host = open(os.path.join(programs_dir, "build", name + ".o.host.cpp")).read()
        assert re.search(r"_block\[3\] = \{\(uint32_t\)\((128|32)\)", host)


@pytest.mark.parametrize("name", sorted(CASES))
def test_cpu_generated_code_matches_numpy(programs_dir, name):
    A, x, expected = inputs(name, True, 1)
    out = np.full((A.shape[0],), 7, A.dtype)
    cpu = runtime.Program(oracle_build.cpu_program_library(programs_dir, name), name, needs_gpu_runtime=False)
    call(cpu, A, x, out)
    assert np.array_equal(out, expected.astype(A.dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_gpu_matches_numpy(programs_dir, name):
    from gpu_util import DeviceArray, assert_fp32_parity
    prog = runtime.load(programs_dir, name)
    for integer in (True,) if name in INT32 else (True, False):
        A, x, expected = inputs(name, integer, 2 + integer)
        out = np.full((A.shape[0],), 7, A.dtype)
        dev = [DeviceArray(a) for a in ([A, out] if x is None else [A, x, out])]
        print("running", name, "integer" if integer else "uniform", flush=True)
        prog(*[d.buffer() for d in dev])
        got = dev[-1].download()
        for d in dev:
            d.free()
        if integer:
            assert np.array_equal(got, expected.astype(A.dtype))
        else:
            assert_fp32_parity(got, expected, name + " vs float64 numpy", 1e-4)


def test_sum_across_wavefronts_under_a_condition_on_the_block_iterator(programs_dir):
    """tests/programs/thread_reduction_under_condition.cpp: the 256-thread loop sits under `if (block iterator >= 3)`.
    The lowering across wavefronts ends in a workgroup barrier that every thread must reach; this condition is the
    same for all threads of a workgroup, so the sum is lowered below it."""
    text = open(os.path.join(programs_dir, "build", "row_sums_from_row_3.o.hip")).read()
    kernel = text[text.index('extern "C" __global__'):]
    assert "if ((c1 >= 3))" in kernel
    assert "block_group_sum<256>" in kernel[kernel.index("if ((c1 >= 3))"):]
    assert "DPP wavefront reductions" in re.search(r"^// _kernel_\d+: (.*)$", text, re.M).group(1)


@pytest.mark.gpu
def test_gpu_sum_under_a_condition_on_the_block_iterator(programs_dir):
    from gpu_util import DeviceArray
    rng = np.random.RandomState(40)
    A = (rng.randint(0, 10, (40, 5000)) - 5).astype(np.float32)
    expected = A.astype(np.float64).sum(axis=1).astype(np.float32)
    expected[:3] = 0
    dev = [DeviceArray(A), DeviceArray(np.full(40, -7.0, np.float32))]
    print("row_sums_from_row_3", flush=True)
    runtime.load(programs_dir, "row_sums_from_row_3")(*[d.buffer() for d in dev])
    got = dev[1].download()
    for d in dev:
        d.free()
    assert np.array_equal(got, expected)


def test_sums_left_as_scheduled_are_reported(programs_dir, tmp_path):
    """tests/programs/thread_reduction_left_as_scheduled.cpp: a bfloat16 sum on the lanes, and an update that lies inside
    one of the kernel's two thread loops only.  The reference emits such code silently
    (tiramisu_codegen_cuda.cpp:549-707); this back-end generates it as scheduled too and says what will happen."""
    import subprocess
    os.makedirs(os.path.join(str(tmp_path), "build"))
    env = dict(os.environ, HIPCC_PATH="/bin/true", TIRAMISU_HOST_CXX="/bin/true")
    r = subprocess.run([os.path.join(programs_dir, "build", "gen_thread_reduction_left_as_scheduled")], cwd=str(tmp_path), env=env,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    assert ("GPU mapping: the sum s over thread loop c3 of row_sums_bf16 is emitted as scheduled, its threads race on _s_init_b1 "
            "(sums of tiramisu_bf16_t are not lowered: those of integers, float and double are)") in r.stdout, r.stdout
    assert ("GPU mapping: bump of update_inside_one_thread_loop_only updates _s_init_b1 from its own value inside some of the "
            "kernel's thread loops only: every thread along dimension x repeats the update") in r.stdout, r.stdout
    assert ("GPU mapping: the sum s over thread loop c3 of row_sums_of_even_columns is emitted as scheduled, its threads race on _s_init_b1 "
            "(the statement carries a predicate or scalar definitions)") in r.stdout, r.stdout
    assert ("GPU mapping: the sum s over thread loop c3 of tile_sums is emitted as scheduled, its threads race on _s_init_b1 "
            "(it runs over several thread loops, or over one that is not on threadIdx.x)") in r.stdout, r.stdout
    # the lowered sum of the second program is not reported
    assert "the sum s over thread loop c5 of update_inside_one_thread_loop_only" not in r.stdout
