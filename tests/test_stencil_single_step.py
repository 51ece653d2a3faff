"""One stencil step out of place (tests/programs/stencil_single_step.cpp): the stencil back-end takes a nest
out(y, x) = f(in(y + dy, x + dx)) whose input and output live in buffers of their own.  Checked against numpy
(brute force over the taps, in the program's order of operations) and against the CPU-generated code of the
same program, bit for bit: the sweep has no reassociation freedom and is compiled without contraction."""
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from tiramisu_amd import runtime

CASES = [("sweep5", 300, 520), ("sweep5", 45, 39), ("wide9", 200, 520), ("wide9", 70, 50)]


def expected_of(kind, grid, out):
    f = np.float32
    want = out.copy()
    if kind == "sweep5":
        c, n, s, w, e = grid[1:-1, 1:-1], grid[:-2, 1:-1], grid[2:, 1:-1], grid[1:-1, :-2], grid[1:-1, 2:]
        want[1:-1, 1:-1] = c * f(0.3) + (((n + s) + w) + e) * f(0.4)
    else:
        c = grid[2:-2, 2:-2]
        far = ((grid[:-4, 2:-2] + grid[4:, 2:-2]) + grid[2:-2, :-4]) + grid[2:-2, 4:]
        diag = grid[1:-3, 3:-1] + grid[3:-1, 1:-3]
        want[2:-2, 2:-2] = (c * f(0.5) + far * f(0.0625)) + diag * f(0.125)
    return want


def inputs(kind, ny, nx):
    rng = np.random.RandomState(ny + nx)
    return rng.uniform(0, 1, (ny, nx)).astype(np.float32), np.full((ny, nx), -1.0, np.float32)


@pytest.mark.parametrize("kind,ny,nx", CASES)
def test_taken_by_the_stencil_emitter(programs_dir, kind, ny, nx):
    text = open(os.path.join(programs_dir, "build", "%s_%dx%d.o.hip" % (kind, ny, nx))).read()
    assert "stencil: 1 time step(s) per launch, radius %d" % (1 if kind == "sweep5" else 2) in text and "out of place" in text


@pytest.mark.parametrize("kind,ny,nx", CASES)
def test_cpu_generated_code_matches_numpy(programs_dir, kind, ny, nx):
    name = "%s_%dx%d" % (kind, ny, nx)
    grid, out = inputs(kind, ny, nx)
    want = expected_of(kind, grid, out)
    runtime.Program(oracle_build.cpu_program_library(programs_dir, name), name, needs_gpu_runtime=False)(grid, out)
    assert np.array_equal(out, want)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,ny,nx", CASES + [("sweep5", 8192, 8192)])
def test_gpu_matches_numpy(programs_dir, product_programs_dir, kind, ny, nx):
    from gpu_util import DeviceArray
    name = "%s_%dx%d" % (kind, ny, nx)
    if ny == 8192:
        programs_dir = product_programs_dir     # the benchmark-sized plane: tiramisu_amd/programs/stencil_sweep.cpp
    grid, out = inputs(kind, ny, nx)
    want = expected_of(kind, grid, out)
    dev = [DeviceArray(grid), DeviceArray(out)]
    print("running", name, flush=True)
    runtime.load(programs_dir, name)(*[d.buffer() for d in dev])
    got = dev[1].download()
    for d in dev:
        d.free()
    assert np.array_equal(got, want)        # cells outside the iteration domain keep what they held
