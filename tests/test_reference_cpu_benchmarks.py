"""The reference's tuned CPU benchmark generators, unchanged, through this front-end and the oracle's CPU emitter
(tests/reference_programs/build_reference_programs.py: CPU_BENCHMARKS): the sgemm with packed operands, three-level
tiling and separated partial tiles, and the direct convolution with blocked layouts whose register tile is named
through a tiramisu::view.  Both against numpy on small integers (exact).  No GPU; skipped where the reference tree
was absent at build time."""
import os
import subprocess
import sys

import numpy as np
import pytest

from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILD = os.path.join(ROOT, "tests", "reference_programs", "build")


def library(name):
    path = os.path.join(BUILD, "lib%s.so" % name)
    if not os.path.exists(path):
        pytest.skip("reference tree was absent when the libraries were built")
    return path


def test_tuned_cpu_sgemm_generator_matches_numpy():
    """benchmarks/linear_algebra/blas/level3/sgemm/cpu/sgemm_generator.cpp: C = a A B + b C with sizes at run time
    (multiples of its tiles, as its configuration asks)."""
    p = runtime.Program(library("sgemm_cpu_tuned"), "sgemm_tiramisu", needs_gpu_runtime=False)
    n = 512
    rng = np.random.RandomState(1)
    A, B, C = (rng.randint(-3, 4, (n, n)).astype(np.float32) for _ in range(3))
    expected = (1.5 * (A.astype(np.float64) @ B) + 0.5 * C).astype(np.float32)
    p(np.array([n, n, n], np.int32), np.array([1.5], np.float32), np.array([0.5], np.float32), A, B, C)
    assert np.array_equal(C, expected)


CONV_CHECK = r'''
import sys
import numpy as np
sys.path.insert(0, %r)
from tiramisu_amd import runtime
BATCH, N, FIn, FOut, K, FINB, FOUTB = 8, 112, 128, 256, 3, 16, 8      # the generator's configure.h
p = runtime.Program(%r, "conv_tiramisu", needs_gpu_runtime=False)
rng = np.random.RandomState(1)
x = rng.randint(-2, 3, (BATCH, FIn, N + 2, N + 2)).astype(np.float32)
w = rng.randint(-2, 3, (FOut, FIn, K, K)).astype(np.float32)
b = rng.randint(-2, 3, (FOut,)).astype(np.float32)
# c_input[n][fin_b][y][x][ffin], filter[fout_b][fin_b][k_y][k_x][ffin][ffout], bias[fout_b][ffout], out[n][fout_b][y][x][ffout]
xin = np.ascontiguousarray(x.reshape(BATCH, FIn // FINB, FINB, N + 2, N + 2).transpose(0, 1, 3, 4, 2))
wf = np.ascontiguousarray(w.reshape(FOut // FOUTB, FOUTB, FIn // FINB, FINB, K, K).transpose(0, 2, 4, 5, 3, 1))
out = np.zeros((BATCH, FOut // FOUTB, N, N, FOUTB), np.float32)
p(xin, wf, np.ascontiguousarray(b.reshape(FOut // FOUTB, FOUTB)), out)
got = out.transpose(0, 1, 4, 2, 3).reshape(BATCH, FOut, N, N)
# whole rows of a few (image, output channel) pairs against a float64 restatement
for n, fo in [(0, 0), (3, 17), (7, 255)]:
    e = np.full((N, N), b[fo], np.float64)
    for ky in range(K):
        for kx in range(K):
            e += np.einsum("c,cyx->yx", w[fo, :, ky, kx].astype(np.float64), x[n, :, ky:ky + N, kx:kx + N])
    assert np.array_equal(got[n, fo], e.astype(np.float32)), (n, fo)
print("ok")
'''


def test_tuned_cpu_convolution_generator_matches_numpy_on_one_thread():
    """benchmarks/DNN/layers/convolution/direct/cpu/conv_layer_generator_tiramisu.cpp at its own configuration (batch 8,
    128 -> 256 features, 112 x 112).  One thread: the program keeps its register tile in one temporary buffer that the
    iterations of its parallel loops share."""
    env = dict(os.environ)
    env["OMP_NUM_THREADS"] = "1"
    r = subprocess.run([sys.executable, "-c", CONV_CHECK % (ROOT, library("conv_cpu_tuned"))], env=env, stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), r.stdout[-2000:]
