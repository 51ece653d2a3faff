"""The Python front-end (tiramisu_amd/python/tiramisu; names and overloads of the reference's
python_bindings/tiramisu.pyi): the module loads and builds expressions without a GPU, and the two
programs written with it (tests/python_programs/*.py, generated at build time) reach the pattern
emitters and compute what the numpy restatements say."""
import os
import re
import sys

import numpy as np
import pytest

from oracle import reference_loops as ref
from tiramisu_amd import build, runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tests", "python_programs")


@pytest.fixture(scope="module")
def tm():
    assert os.path.exists(build.python_module()), "run __graft_entry__.build() first"
    sys.path.insert(0, os.path.join(ROOT, "tiramisu_amd", "python"))
    try:
        import tiramisu
    finally:
        sys.path.pop(0)
    return tiramisu


def test_names_of_the_reference_stub_are_present(tm):
    for name in ["init", "codegen", "pycodegen", "memcpy", "allocate", "cuda_stream_synchronize", "get_implicit_function",
                 "expr", "var", "sync", "buffer", "computation", "input", "constant", "function",
                 "primitive_t", "argument_t", "op_t", "expr_t", "hardware_architecture_t",
                 "p_float32", "p_uint8", "a_input", "a_output", "a_temporary", "o_max", "o_expo", "arch_nvidia_gpu"]:
        assert hasattr(tm, name), name
    for method in ["after", "after_low_level", "cache_shared", "dump", "get_buffer", "gpu_tile", "parallelize", "set_expression",
                   "split", "store_in", "then", "tile", "__getitem__"]:
        assert hasattr(tm.computation, method), method


def test_expressions_and_schedules_from_python(tm):
    tm.init("python_front_end_check")
    i, j = tm.var("i", 0, 8), tm.var("j", 0, 8)
    A = tm.input("A", [i, j], tm.primitive_t.p_int32)
    e = A[i, j] * 2 + 3 - i % 4
    assert str(e) == "(((A(i, j) * 2) + 3) - (i % 4))"
    assert tm.expr(7).get_int32_value() == 7 and tm.expr(2.5).get_float32_value() == 2.5
    assert str(tm.expr(tm.op_t.o_max, A[i, j], tm.expr(0))) == "max(A(i, j), 0)"
    C = tm.computation("C", [i, j], e)
    i0, j0, i1, j1 = tm.var("i0"), tm.var("j0"), tm.var("i1"), tm.var("j1")
    C.gpu_tile(i, j, 4, 4, i0, j0, i1, j1)
    assert C.get_buffer().get_name() == "_C_b0" or C.get_buffer().get_name()   # an automatic buffer exists
    assert tm.get_implicit_function().get_name() == "python_front_end_check"


@pytest.mark.parametrize("name,kind", [("sgemm_py", "mfma-contraction"), ("heat2d_py", "stencil")])
def test_python_programs_reach_the_pattern_emitters(name, kind):
    text = open(os.path.join(PROGRAMS, "build", name + ".o.hip")).read()
    assert re.search(r"^// _kernel_\d+: " + kind, text, re.M)


@pytest.mark.gpu
def test_sgemm_written_in_python():
    from gpu_util import DeviceArray
    M, N, K = 192, 128, 96
    rng = np.random.RandomState(192)
    A = rng.randint(-4, 5, (M, K)).astype(np.float32)
    B = rng.randint(-4, 5, (K, N)).astype(np.float32)
    C = rng.randint(-4, 5, (M, N)).astype(np.float32)
    expected = ref.sgemm(A, B, C, 3.0, 2.0)
    dA, dB, dC = DeviceArray(A), DeviceArray(B), DeviceArray(C)
    runtime.load(PROGRAMS, "sgemm_py")(np.array([3.0, 2.0], np.float32), dA.buffer(), dB.buffer(), dC.buffer())
    assert np.array_equal(dC.download(), expected)


@pytest.mark.gpu
def test_heat2d_written_in_python():
    from gpu_util import DeviceArray
    N, STEPS = 130, 5
    grid = np.zeros((N, N), np.float32)
    grid[1:-1, 1:-1] = np.random.RandomState(130).uniform(0, 1, (N - 2, N - 2)).astype(np.float32)
    planes = np.zeros((2, N, N), np.float32)
    planes[0] = grid
    d = DeviceArray(planes)
    runtime.load(PROGRAMS, "heat2d_py")(d.buffer())
    assert np.array_equal(d.download(), ref.heat2d(grid, STEPS))


def test_every_name_of_the_reference_stub_exists(tm):
    """Classes, their methods and the module's functions of the reference's python_bindings/tiramisu.pyi (read
    where it lies; skipped where the tree is absent) exist in this module under the same names."""
    stub = "/root/reference/python_bindings/tiramisu.pyi"
    if not os.path.exists(stub):
        pytest.skip("reference tree absent")
    t = tm
    missing, current = [], None
    for line in open(stub):
        m = re.match(r"^class ([A-Za-z_0-9]+)", line)
        if m:
            current = m.group(1)
            if not hasattr(t, current):
                missing.append(current)
            continue
        m = re.match(r"^    def ([a-zA-Z_][a-zA-Z_0-9]*)", line)
        if m and current and hasattr(t, current) and not m.group(1).startswith("__") and not hasattr(getattr(t, current), m.group(1)):
            missing.append(current + "." + m.group(1))
        m = re.match(r"^def ([a-zA-Z_][a-zA-Z_0-9]*)", line)
        if m and not hasattr(t, m.group(1)):
            missing.append(m.group(1))
    assert not missing, sorted(set(missing))
