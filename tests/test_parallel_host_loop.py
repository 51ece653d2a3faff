"""Host loops tagged parallel around GPU kernels (tests/programs/parallel_host_loop.cpp).  Left alone, the HIP
back-end distributes such a loop over its statements: every kernel once with the iterations as gridDim.z, library
GEMM calls of a statement gathered into one batched launch (tiramisu_hip_batch_begin / _end).  With that switched
off it hands the loop body to tiramisu_hip_parallel_for, whose pool threads launch on streams of their own.
Exact arithmetic (small integers), compared with numpy and with the same program generated with a serial loop."""
import os

import numpy as np
import pytest

from tiramisu_amd import runtime


def test_loop_is_handed_to_the_pool(programs_dir):
    threaded = open(os.path.join(programs_dir, "build", "parallel_host_loop.o.host.cpp")).read()
    serial = open(os.path.join(programs_dir, "build", "parallel_host_loop_serial.o.host.cpp")).read()
    assert "tiramisu_hip_parallel_for(0, 5," in threaded
    assert "tiramisu_hip_parallel_for" not in serial


def test_loop_is_distributed_over_its_kernels(programs_dir):
    host = open(os.path.join(programs_dir, "build", "parallel_host_loop_distributed.o.host.cpp")).read()
    device = open(os.path.join(programs_dir, "build", "parallel_host_loop_distributed.o.hip")).read()
    assert "tiramisu_hip_parallel_for" not in host and "distributed over its statements" in host
    assert host.count("const int32_t _batch_first = 0;") == 2                 # the two kernels of the body, once each
    assert device.count("= (int32_t)blockIdx.z + _batch_first;") == 2
    import json
    m = json.load(open(os.path.join(programs_dir, "build", "parallel_host_loop.o.json")))
    assert {"name": "hip_no_distributed_host_loops", "value": "1", "from": "program"} in m["options"]


@pytest.mark.gpu
def test_parallel_iterations_match_numpy_and_the_serial_loop(programs_dir):
    from gpu_util import DeviceArray
    P, N = 6, 256
    rng = np.random.RandomState(6)
    src = rng.randint(-4, 5, (N, N)).astype(np.float32)
    base = src + 1
    expected = np.zeros((N, N), np.float32)
    for p in range(P):
        s1 = base * (p + 1)
        expected += s1 + s1[::-1]
    outs = {}
    for name in ("parallel_host_loop", "parallel_host_loop_distributed", "parallel_host_loop_serial"):
        program = runtime.load(programs_dir, name)
        for repeat in range(3):                      # the pool is reused from call to call
            d_in, d_out = DeviceArray(src), DeviceArray(np.full((N, N), -1, np.float32))
            program(d_in.buffer(), d_out.buffer())
            outs[name] = d_out.download()
            assert np.array_equal(outs[name], expected), (name, repeat)


@pytest.mark.gpu
def test_pool_runs_every_iteration_once_and_nested_calls_inline():
    import ctypes
    w = runtime.wrappers()
    body_t = ctypes.CFUNCTYPE(None, ctypes.c_int32, ctypes.c_void_p)
    w.tiramisu_hip_parallel_for.argtypes = [ctypes.c_int32, ctypes.c_int32, body_t, ctypes.c_void_p]
    w.tiramisu_hip_parallel_for.restype = None
    counts = np.zeros(40, np.int64)
    inner = np.zeros((40, 3), np.int64)

    def nested(k, closure):
        inner[closure or 0, k] += 1

    def body(i, _):
        counts[i - 5] += 1
        w.tiramisu_hip_parallel_for(0, 2, body_t(nested), ctypes.c_void_p(i - 5))

    w.tiramisu_hip_parallel_for(5, 44, body_t(body), None)
    assert np.all(counts == 1) and np.all(inner == 1)
    w.tiramisu_hip_parallel_for(3, 2, body_t(body), None)      # empty range: nothing runs
    assert np.all(counts == 1)
