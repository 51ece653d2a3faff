"""A triangular domain under gpu_tile (tests/programs/triangular_domain.cpp): the bound of one block loop is a function
of another block loop's iterator alone.  The grid must cover the whole range of that bound, a guard in the kernel must
cut the triangle out, and the elements above the diagonal stay untouched."""
import os
import re

import numpy as np
import pytest

from oracle import build as oracle_build
from tiramisu_amd import runtime

CASES = [("lower_triangle_16x16", 106, (7, 7)), ("lower_triangle_16x4", 45, (12, 3))]


def inputs_and_expected(n):
    rng = np.random.RandomState(n)
    a = rng.randint(-9, 10, (n, n)).astype(np.int32)
    e = np.full((n, n), -777, np.int32)
    lower = np.tril(np.ones((n, n), bool))
    e[lower] = (a + 2 * a.T)[lower]
    return a, e


@pytest.mark.parametrize("name, n, grid", CASES)
def test_the_grid_covers_the_range_of_the_dependent_bound(programs_dir, name, n, grid):
    host = open(os.path.join(programs_dir, "build", name + ".o.host.cpp")).read()
    m = re.search(r"_grid\[3\] = \{\(uint32_t\)\((\d+)\), \(uint32_t\)\((\d+)\), \(uint32_t\)\(1\)\}", host)
    assert m and (int(m.group(1)), int(m.group(2))) == grid, host[:2000]
    kernel = open(os.path.join(programs_dir, "build", name + ".o.hip")).read()
    assert re.search(r"if \(c3 >= 0 && c3 <= ", kernel)            # the guard that names the other block iterator


@pytest.mark.parametrize("name, n, grid", CASES)
def test_cpu_emitter_on_the_triangle(programs_dir, name, n, grid):
    a, e = inputs_and_expected(n)
    out = np.full((n, n), -777, np.int32)
    runtime.Program(oracle_build.cpu_program_library(programs_dir, name), name, needs_gpu_runtime=False)(a, out)
    assert np.array_equal(out, e)


@pytest.mark.gpu
@pytest.mark.parametrize("name, n, grid", CASES)
def test_triangle_on_the_gpu(programs_dir, name, n, grid):
    from gpu_util import DeviceArray
    a, e = inputs_and_expected(n)
    da, do = DeviceArray(a), DeviceArray(np.full((n, n), -777, np.int32))
    print(name, flush=True)
    runtime.load(programs_dir, name)(da.buffer(), do.buffer())
    got = do.download()
    da.free()
    do.free()
    assert np.array_equal(got, e)
