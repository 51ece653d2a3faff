"""Time-tiled stencil back-end on stencils other than heat2d: diagonal taps, radius 2, rectangular
planes, two planes with different fixed boundaries.  Bit for bit against the CPU-generated code and
the numpy restatement (no reassociation freedom: same fp32 operations in the same order)."""
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from oracle import reference_loops as ref
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tests", "programs")
BOX9 = [(200, 520, 6), (45, 39, 3)]
FAR2 = [(200, 520, 5), (70, 50, 4)]
BOX9_TAPS = [(0.25, [(0, 0)]), (0.125, [(-1, 0), (1, 0), (0, -1), (0, 1)]),
             (0.0625, [(-1, -1), (-1, 1), (1, -1), (1, 1)])]
FAR2_TAPS = [(0.5, [(0, 0)]), (0.0625, [(-2, 0), (2, 0), (0, -2), (0, 2)]), (0.125, [(-1, 1), (1, -1)])]
CASES = [("box9", ref.stencil_box9, c) for c in BOX9] + [("far2", ref.stencil_far2, c) for c in FAR2]


def random_planes(ny, nx, seed):
    # both planes random: fixed boundary cells differ between the planes
    return np.random.RandomState(seed).uniform(0.0, 1.0, (2, ny, nx)).astype(np.float32)


def test_oracle_matches_brute_force():
    p = random_planes(9, 11, 1)
    assert np.array_equal(ref.stencil_box9(p, 3), ref.stencil_loops(p, 3, 1, BOX9_TAPS))
    assert np.array_equal(ref.stencil_far2(p, 3), ref.stencil_loops(p, 3, 2, FAR2_TAPS))


def test_oracle_weights_preserve_a_constant_field():
    # both weight sets sum to one in exactly representable steps
    p = np.full((2, 12, 14), 3.0, np.float32)
    assert np.all(ref.stencil_box9(p, 4) == 3.0)
    assert np.all(ref.stencil_far2(p, 4) == 3.0)


def test_oracle_single_cell_footprint():
    p = np.zeros((2, 11, 11), np.float32)
    p[0, 5, 5] = 16.0
    o = ref.stencil_far2(p, 1)[1]
    assert o[5, 5] == 8.0 and o[3, 5] == o[7, 5] == o[5, 3] == o[5, 7] == 1.0
    # a tap at (dy, dx) of the output reads the hot cell when the output sits at (-dy, -dx) of it
    assert o[6, 4] == 2.0 and o[4, 6] == 2.0 and o[4, 4] == 0.0 and o[6, 6] == 0.0
    assert np.count_nonzero(o) == 7


@pytest.mark.parametrize("kind,oracle,case", CASES)
def test_cpu_generated_code_matches_oracle(kind, oracle, case):
    ny, nx, steps = case
    name = "%s_%dx%dx%d" % (kind, ny, nx, steps)
    p = random_planes(ny, nx, ny + steps)
    out = p.copy()
    runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)(out)
    assert np.array_equal(out, oracle(p, steps))


@pytest.mark.gpu
@pytest.mark.parametrize("kind,oracle,case", CASES)
def test_gpu_matches_oracle(kind, oracle, case):
    ny, nx, steps = case
    name = "%s_%dx%dx%d" % (kind, ny, nx, steps)
    p = random_planes(ny, nx, 3 * ny + steps)
    w = runtime.wrappers()
    dev = w.tiramisu_hip_malloc(p.nbytes)
    w.tiramisu_hip_memcpy_to_device(dev, p.ctypes.data, p.nbytes)
    runtime.load(PROGRAMS, name)(runtime.Buffer.from_device(dev, p.shape, np.float32))
    w.tiramisu_hip_stream_synchronize(0)
    out = np.empty_like(p)
    w.tiramisu_hip_memcpy_to_host(out.ctypes.data, dev, p.nbytes)
    w.tiramisu_hip_free(dev)
    assert np.array_equal(out, oracle(p, steps))
