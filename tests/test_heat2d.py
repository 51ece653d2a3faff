"""heat2d (benchmark configuration 2): oracle pins, CPU-generated code vs the oracle, and the time-tiled
HIP stencil kernel vs both -- bit for bit (the sweep has no reassociation freedom: every cell
is the same five fp32 additions and one multiplication on every path)."""
import ctypes
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from oracle import reference_loops as ref
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")
SMALL = [(256, 1), (130, 4), (66, 7), (37, 6), (20, 2)]


def initial_grid(n, seed):
    rng = np.random.RandomState(seed)
    g = np.zeros((n, n), np.float32)
    g[1:-1, 1:-1] = rng.uniform(0.0, 1.0, (n - 2, n - 2)).astype(np.float32)
    return g


def cpu_program(n, steps):
    name = "heat2d_%dx%d" % (n, steps)
    return runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)


# ---------------------------------------------------------------- oracle pins (no GPU)

def test_launch_plan_of_the_full_size_program():
    """32 steps are three launches: odd chunks between the two planes, the last of them into a third plane,
    and a final launch that writes the last step and the last but one into the two planes."""
    import json
    import re
    base = os.path.join(PROGRAMS, "build", "heat2d_8192x32.o")
    ranges = [(int(a), int(b)) for a, b in re.findall(r"_st_src = \d+;  // steps (\d+)\.\.(\d+)", open(base + ".host.cpp").read())]
    assert ranges[0][0] == 1 and ranges[-1][1] == 32 and len(ranges) == 3
    assert all(a[1] + 1 == b[0] for a, b in zip(ranges, ranges[1:]))
    assert all((b - a + 1) % 2 == 1 for a, b in ranges[:-1])
    hows = [k["how"] for k in json.load(open(base + ".json"))["kernels"] if "interior tiles" in k["how"]]
    assert sum("into a third plane" in h and "from" not in h for h in hows) == 1
    assert sum("from a third plane into both planes" in h for h in hows) == 1


def test_oracle_matches_python_loops():
    g = initial_grid(9, 1)
    assert np.array_equal(ref.heat2d(g, 3), ref.heat2d_loops(g, 3))


def test_oracle_closed_forms():
    n = 12
    ones = np.ones((n, n), np.float32)
    ones[0, :] = ones[-1, :] = ones[:, 0] = ones[:, -1] = 0
    out = ref.heat2d(ones, 1)[1]
    # away from the boundary five ones average to exactly one; next to an edge one neighbour is 0
    assert np.all(out[2:-2, 2:-2] == np.float32(1.0))
    assert np.all(out[1, 2:-2] == np.float32(4.0) * np.float32(0.2))
    assert np.all(out[0, :] == 0) and np.all(out[:, 0] == 0)
    # a single hot cell spreads to its four neighbours only, symmetrically
    delta = np.zeros((n, n), np.float32)
    delta[5, 6] = 5.0
    o = ref.heat2d(delta, 1)[1]
    assert o[5, 6] == o[4, 6] == o[6, 6] == o[5, 5] == o[5, 7] == np.float32(1.0)
    assert np.count_nonzero(o) == 5
    # the grid transposed gives the transposed result (w/e and n/s terms are added in a fixed
    # order, so this holds to rounding only)
    g = initial_grid(n, 3)
    assert np.allclose(ref.heat2d(g.T.copy(), 4)[0], ref.heat2d(g, 4)[0].T, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("n,steps", SMALL)
def test_cpu_generated_code_matches_oracle(n, steps):
    g = initial_grid(n, n + steps)
    planes = np.zeros((2, n, n), np.float32)
    planes[0] = g
    cpu_program(n, steps)(planes)
    assert np.array_equal(planes, ref.heat2d(g, steps))


# ---------------------------------------------------------------- GPU parity

def run_on_gpu(n, steps, planes):
    w = runtime.wrappers()
    nbytes = planes.nbytes
    dev = w.tiramisu_hip_malloc(nbytes)
    w.tiramisu_hip_memcpy_to_device(dev, planes.ctypes.data, nbytes)
    name = "heat2d_%dx%d" % (n, steps)
    prog = runtime.load(PROGRAMS, name)
    prog(runtime.Buffer.from_device(dev, planes.shape, np.float32))
    w.tiramisu_hip_stream_synchronize(0)
    out = np.empty_like(planes)
    w.tiramisu_hip_memcpy_to_host(out.ctypes.data, dev, nbytes)
    w.tiramisu_hip_free(dev)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("n,steps", SMALL + [(1024, 8), (1030, 9)])
def test_gpu_matches_oracle(n, steps):
    g = initial_grid(n, 7 * n + steps)
    planes = np.zeros((2, n, n), np.float32)
    planes[0] = g
    out = run_on_gpu(n, steps, planes)
    assert np.array_equal(out, ref.heat2d(g, steps))


@pytest.mark.gpu
@pytest.mark.parametrize("n,steps", [(66, 7), (130, 4), (1030, 9), (20, 2)])
def test_gpu_boundaries_of_both_planes_are_respected(n, steps):
    # the two planes hold different fixed boundary values: even steps read plane 1's boundary (with three
    # steps or more the launches go through a third plane, which has to show the right plane's fixed cells)
    rng = np.random.RandomState(5)
    planes = rng.uniform(0, 1, (2, n, n)).astype(np.float32)
    expected = ref.heat2d(planes[0], steps, boundary_other=planes[1])
    out = run_on_gpu(n, steps, planes.copy())
    assert np.array_equal(out, expected)


@pytest.mark.gpu
def test_gpu_full_size_matches_cpu_generated_code():
    # benchmark size: 8192 x 8192, 32 steps.  Two checkers, both planes compared bit for bit: the
    # CPU-generated code (parallelize y, vectorize x), which shares the front-end with the GPU path,
    # and the numpy restatement, which shares nothing with it.
    n, steps = 8192, 32
    g = initial_grid(n, 8192)
    planes = np.zeros((2, n, n), np.float32)
    planes[0] = g
    out = run_on_gpu(n, steps, planes)
    assert np.array_equal(out, ref.heat2d(g, steps))
    cpu_program(n, steps)(planes)
    assert np.array_equal(out, planes)
    assert np.all(out[:, 0, :] == 0) and np.all(out[:, :, -1] == 0)
