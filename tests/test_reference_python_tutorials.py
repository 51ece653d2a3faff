"""The reference's Python tutorials (python_bindings/tutorials/tutorial_01 ... tutorial_05.py), unchanged, through this
build's Python front-end (tiramisu_amd/csrc/python_module.cpp, names and overloads of python_bindings/tiramisu.pyi).
They are CPU programs: the object each one generates comes from the oracle's CPU emitter, registered by the
runner (tests/reference_programs/run_python_tutorial.py), is linked into a shared library here and called on seeded
data; the expectations are what the tutorials' own comments state, restated in numpy."""
import os
import subprocess
import sys

import numpy as np
import pytest

from oracle import build as oracle_build
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = os.environ.get("TIRAMISU_REFERENCE_TREE", "/root/reference")
TUTORIALS = os.path.join(REFERENCE, "python_bindings", "tutorials")
RUNNER = os.path.join(ROOT, "tests", "reference_programs", "run_python_tutorial.py")

pytestmark = pytest.mark.skipif(not os.path.isdir(TUTORIALS) or not os.path.exists(oracle_build.CPU_BACKEND),
                                reason="needs the reference's tutorials and the oracle's CPU emitter")


def run_tutorial(name, tmp_path):
    r = subprocess.run([sys.executable, RUNNER, os.path.join(TUTORIALS, name + ".py")], cwd=str(tmp_path),
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-3000:]
    return r.stdout


def generated(tmp_path, obj, function):
    lib = os.path.join(str(tmp_path), "lib_" + function + ".so")
    subprocess.run(["g++", "-shared", "-fopenmp", "-o", lib, os.path.join(str(tmp_path), obj)], check=True)
    return runtime.Program(lib, function, needs_gpu_runtime=False)


def test_tutorial_01_a_constant_for_every_iteration(tmp_path):
    run_tutorial("tutorial_01", tmp_path)
    out = np.zeros(20, np.uint8)             # S0 runs over N = 20 iterations
    generated(tmp_path, "generated_fct_developers_tutorial_01.o", "test")(out)
    assert np.array_equal(out, np.full(20, 7, np.uint8))


def test_tutorial_01_A_pycodegen_makes_an_importable_module(tmp_path):
    out = run_tutorial("tutorial_01_A", tmp_path)
    assert "[7 7 7 7 7 7 7 7 7 7 7 7 7 7 7 7 7 7 7 7]" in out


def test_tutorial_02_tiled_and_parallel(tmp_path):
    run_tutorial("tutorial_02", tmp_path)
    rng = np.random.RandomState(2)
    A = rng.randint(0, 200, (10, 20)).astype(np.uint8)
    out = np.zeros((10, 20), np.uint8)
    generated(tmp_path, "generated_fct_developers_tutorial_02.o", "tut_02")(A, out)
    expected = (A.astype(np.int64) + np.arange(10)[:, None] + 4).astype(np.uint8)
    assert np.array_equal(out, expected)


def test_tutorial_03_order_of_four_computations(tmp_path):
    run_tutorial("tutorial_03", tmp_path)
    b0, b1, b3 = (np.full(10, 99, np.uint8) for _ in range(3))
    b2 = np.full((10, 10), 99, np.uint8)
    generated(tmp_path, "generated_fct_developers_tutorial_03.o", "sequence")(b0, b1, b2, b3)
    assert (b0 == 4).all() and (b1 == 3).all() and (b2 == 2).all() and (b3 == 1).all()


def matmul_u8(A, B):
    return (A.astype(np.int64) @ B.astype(np.int64)).astype(np.uint8)       # uint8 arithmetic wraps


def test_tutorial_04A_matmul(tmp_path):
    run_tutorial("tutorial_04A", tmp_path)
    rng = np.random.RandomState(4)
    A, B = rng.randint(0, 256, (100, 100)).astype(np.uint8), rng.randint(0, 256, (100, 100)).astype(np.uint8)
    C = np.full((100, 100), 99, np.uint8)
    generated(tmp_path, "generated_fct_developers_tutorial_04A.o", "matmul")(A, B, C)
    assert np.array_equal(C, matmul_u8(A, B))


def test_tutorial_04B_two_fused_matmuls(tmp_path):
    run_tutorial("tutorial_04B", tmp_path)
    rng = np.random.RandomState(5)
    A, B, D = (rng.randint(0, 256, (100, 100)).astype(np.uint8) for _ in range(3))
    C, E = np.full((100, 100), 99, np.uint8), np.full((100, 100), 99, np.uint8)
    generated(tmp_path, "generated_fct_developers_tutorial_04B.o", "matmul")(A, B, C, D, E)
    assert np.array_equal(C, matmul_u8(A, B)) and np.array_equal(E, matmul_u8(A, D))


def test_tutorial_05_function_objects(tmp_path):
    assert run_tutorial("tutorial_05", tmp_path).strip().endswith("a")
