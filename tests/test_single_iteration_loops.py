"""GPU-tagged loops that all have a single iteration (tests/python_programs/single_iteration_loops.py): isl's AST
holds no loop node for them, and the reference leaves the case open (tiramisu_codegen_cuda.cpp:252, "TODO check if
degenerate").  The statements must still end up in a kernel of one workgroup: fused statements in the same one, a host
loop outside the tagged levels around the launch."""
import os
import re

import numpy as np
import pytest

from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tests", "python_programs")


def generated(name, suffix):
    return open(os.path.join(PROGRAMS, "build", name + suffix)).read()


def test_fused_statements_of_a_single_point_share_one_kernel():
    text = generated("single_point_py", ".o.hip")
    kernels = re.findall(r"__global__ void __launch_bounds__\((\d+)\) (_kernel_\d+)", text)
    assert len(kernels) == 1 and kernels[0][0] == "1"
    body = text[text.index("__global__"):]
    assert body.index("tb[0] =") < body.index("o[0] =")
    host = generated("single_point_py", ".o.host.cpp")
    assert "tb[0] =" not in host and "o[0] =" not in host          # nothing of it runs on the host


def test_a_host_loop_outside_the_tagged_levels_stays_around_the_launch():
    text = generated("single_point_steps_py", ".o.hip")
    assert re.search(r"__global__ void __launch_bounds__\(1\) _kernel_\d+\(const int32_t c1, ", text)
    assert "for (" not in text[text.index("__global__"):]
    host = generated("single_point_steps_py", ".o.host.cpp")
    assert re.search(r"for \(int32_t c1 = 0; c1 <= 4; c1 \+= 1\)", host)


@pytest.mark.gpu
def test_single_point_programs_on_the_gpu():
    from gpu_util import DeviceArray
    a = np.array([[7]], np.int32)
    da, do = DeviceArray(a), DeviceArray(np.full((1, 1), -1, np.int32))
    print("single_point_py", flush=True)
    runtime.load(PROGRAMS, "single_point_py")(da.buffer(), do.buffer())
    assert do.download()[0, 0] == 8 * 8 - 7
    a = np.array([3, -4, 5, 0, 11], np.int32)
    da, do = DeviceArray(a), DeviceArray(np.full(5, -1, np.int32))
    print("single_point_steps_py", flush=True)
    runtime.load(PROGRAMS, "single_point_steps_py")(da.buffer(), do.buffer())
    assert np.array_equal(do.download(), a * 2 + np.arange(5, dtype=np.int32))
