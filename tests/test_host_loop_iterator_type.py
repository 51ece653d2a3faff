"""Kernels that take an iterator of a host loop as a parameter, in a program with 64-bit loop iterators
(tests/programs/host_loop_iterator_int64.cpp; global::set_loop_iterator_type, which the reference's tensor benchmarks
use): the launch passes the address of the generated loop's variable, so the kernel's parameter must have that
variable's width.  Generated code is inspected on the CPU and run on the GPU against numpy."""
import os
import re

import numpy as np
import pytest

from tiramisu_amd import runtime

NAMES = ["host_loop_iterator_int64", "host_loop_iterator_int64_parallel"]


@pytest.mark.parametrize("name", NAMES)
def test_scalar_parameters_have_the_width_of_the_host_variables(programs_dir, name):
    hip = open(os.path.join(programs_dir, "build", name + ".o.hip")).read()
    host = open(os.path.join(programs_dir, "build", name + ".o.host.cpp")).read()
    kernels = re.findall(r'extern "C" __global__ void (?:__launch_bounds__\(\d+\) )?(\w+)\(([^)]*)\)', hip)
    assert kernels
    checked = 0
    for kernel, params in kernels:
        scalars = [p.split() for p in params.split(", ") if "*" not in p]          # ['const', 'int32_t', 'c1']
        for _, ctype, var in scalars:
            declared = re.search(r"\b(?:const )?(\w+) %s = " % re.escape(var), host)
            assert declared, "%s of %s is not declared by the host code" % (var, kernel)
            assert declared.group(1) == ctype, "%s: the host declares %s %s, the kernel takes %s" % (kernel, declared.group(1), var, ctype)
            checked += 1
    assert checked >= 1


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_gpu_matches_numpy(programs_dir, name):
    from gpu_util import DeviceArray
    P, N = 5, 128
    rng = np.random.RandomState(9)
    src = (rng.randint(0, 20, (N, N)) - 10).astype(np.float32)
    expected = np.stack([src * (p + 1) + p for p in range(P)]).astype(np.float32)
    dev = [DeviceArray(src), DeviceArray(np.full((P, N, N), -7.0, np.float32))]
    print("running", name, flush=True)
    runtime.load(programs_dir, name)(*[d.buffer() for d in dev])
    got = dev[1].download()
    for d in dev:
        d.free()
    assert np.array_equal(got, expected)
