"""Contractions with a sliding-window operand in shapes other than the benchmark's convolution
(tests/programs/window_contractions.cpp): 1-D with 9 taps, 5x5 over rectangular images with two tile rows, a launch
whose last tiles are cut into pieces, blocks of 4 channels.  Integer-valued data: the GPU result must equal numpy's
exactly, and the CPU-generated code's."""
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tests", "programs")

# name -> (batch, channels in, channels out, image shape, taps shape)
CASES = {"window_conv1d_9": (6, 16, 64, (1024,), (9,)), "window_conv2d_5x5": (3, 8, 128, (24, 32), (5, 5)),
         "window_conv2d_3x3_pieces": (129, 16, 64, (32, 32), (3, 3)), "window_conv2d_3x3_c4": (2, 4, 64, (16, 16), (3, 3))}


def inputs(name, seed):
    nb, ci, co, image, taps = CASES[name]
    rng = np.random.RandomState(seed)
    padded = tuple(s + t - 1 for s, t in zip(image, taps))
    x = rng.randint(-3, 4, (nb, ci) + padded).astype(np.float32)
    w = rng.randint(-2, 3, (co, ci) + taps).astype(np.float32)
    b = rng.randint(-5, 6, (co,)).astype(np.float32)
    return x, w, b


def expected(name, x, w, b):
    nb, ci, co, image, taps = CASES[name]
    out = np.zeros((nb, co) + image, np.float64) + b.reshape((1, co) + (1,) * len(image))
    for t in np.ndindex(*taps):
        window = x[(slice(None), slice(None)) + tuple(slice(o, o + s) for o, s in zip(t, image))].astype(np.float64)
        out += np.einsum("nc...,oc->no...", window, w[(slice(None), slice(None)) + t].astype(np.float64))
    return out.astype(np.float32)


def test_kernels_are_the_windowed_ones():
    for name, how in [("window_conv1d_9", "sliding window of 9 taps staged in LDS by blocks of 8 channels"),
                      ("window_conv2d_5x5", "sliding window of 25 taps"), ("window_conv2d_3x3_pieces", "the last tiles cut into 2 pieces"),
                      ("window_conv2d_3x3_c4", "by blocks of 4 channels")]:
        kernels = runtime.manifest_of(os.path.join(PROGRAMS, "build", "lib%s.so" % name), name)["kernels"]
        assert len(kernels) == 1 and how in kernels[0]["how"], kernels


@pytest.mark.parametrize("name", ["window_conv1d_9", "window_conv2d_3x3_c4"])
def test_cpu_generated_code(name):
    x, w, b = inputs(name, 5)
    out = np.zeros(expected(name, x, w, b).shape, np.float32)
    runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)(x, w, b, out)
    assert np.array_equal(out, expected(name, x, w, b))


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_gpu_equals_numpy(name):
    from gpu_util import DeviceArray
    prog = runtime.load(PROGRAMS, name)
    for seed in (1, 2):                           # two calls: the launch's queue counters must be left ready for the next
        x, w, b = inputs(name, seed)
        want = expected(name, x, w, b)
        out = np.full(want.shape, -1.0, np.float32)
        d = [DeviceArray(a) for a in (x, w, b, out)]
        print("running", name, "seed", seed, flush=True)
        prog(*[q.buffer() for q in d])
        got = d[3].download()
        for q in d:
            q.free()
        assert np.array_equal(got, want)
