"""tiramisu_hip_sgemm_static_scratch, the entry point that allocates nothing: called through the C ABI
and compared with tiramisu_hip_sgemm (the same kernels, its scratch from hipMalloc) -- bit for bit, on
two calls in a row, the second with a smaller input (the static array keeps the first call's
contents) -- and with a float64 product.  Shapes are deep reductions, whose K range is split over
workgroups through the scratch; one shape that does not split, and one whose split the static
array cannot hold (refused with return value 1, nothing written)."""
import ctypes

import numpy as np
import pytest

from tiramisu_amd import runtime

pytestmark = pytest.mark.gpu


def call(fn, A, B, C, M, N, K, alpha, beta, tA=False, tB=False):
    from gpu_util import DeviceArray
    dA, dB, dC = DeviceArray(A), DeviceArray(B), DeviceArray(C)
    rc = fn(dA.ptr, dB.ptr, dC.ptr, M, N, K, alpha, beta, 0, 0, 0, 0, 0, 0, tA, tB)
    out = dC.download()
    for d in (dA, dB, dC):
        d.free()
    return rc, out


def operands(M, N, K, seed, integer, tA=False, tB=False):
    rng = np.random.RandomState(seed)
    draw = (lambda s: rng.randint(-3, 4, s).astype(np.float32)) if integer else (lambda s: rng.uniform(-1, 1, s).astype(np.float32))
    return draw((K, M) if tA else (M, K)), draw((N, K) if tB else (K, N)), draw((M, N))


def check_pair(M, N, K, seed, tA=False, tB=False):
    w = runtime.wrappers()
    from gpu_util import assert_fp32_parity
    for integer in (True, False):
        A, B, C = operands(M, N, K, seed, integer, tA, tB)
        print("static scratch", M, N, K, "integer" if integer else "uniform", tA, tB, flush=True)
        rc0, expected = call(w.tiramisu_hip_sgemm, A, B, C, M, N, K, 1.5, 0.5, tA, tB)
        rc1, got = call(w.tiramisu_hip_sgemm_static_scratch, A, B, C, M, N, K, 1.5, 0.5, tA, tB)
        assert rc0 == 0 and rc1 == 0
        assert np.array_equal(got, expected)
        exact = 1.5 * ((A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64)) + 0.5 * C
        if integer:
            assert np.array_equal(got, exact.astype(np.float32))
        else:
            assert_fp32_parity(got, exact, "sgemm_static_scratch %dx%dx%d vs float64" % (M, N, K), 1e-4)


def test_two_calls_in_a_row_the_second_smaller():
    check_pair(256, 256, 8192, seed=1)          # 16 tiles x 16 chunks of 512
    check_pair(128, 192, 4096, seed=2)          # 6 tiles x 8 chunks: reuses the array's first part
    check_pair(100, 70, 2500, seed=3)           # ragged tiles, ragged last chunk
    check_pair(192, 64, 4096, seed=4, tA=True, tB=True)


def test_the_static_scratch_call_takes_no_workspace_block():
    """In a thread of its own (the allocating entry point keeps its scratch per thread and stream, so a new thread
    starts without any): a deep reduction through the static-scratch entry point leaves the thread without a
    workspace block, the same shape through tiramisu_hip_sgemm creates one -- the static path did not fall through
    to the allocating one."""
    import threading
    w = runtime.wrappers()
    seen = {}

    def body():
        M, N, K = 128, 128, 4096
        A, B, C = operands(M, N, K, 7, True)
        rc, got = call(w.tiramisu_hip_sgemm_static_scratch, A, B, C, M, N, K, 1.0, 0.0)
        seen["static"] = (rc, w.tiramisu_hip_sgemm_workspace(), got)
        rc, expected = call(w.tiramisu_hip_sgemm, A, B, C, M, N, K, 1.0, 0.0)
        seen["allocating"] = (rc, w.tiramisu_hip_sgemm_workspace(), expected)
    t = threading.Thread(target=body)
    t.start()
    t.join()
    assert seen["static"][0] == 0 and not seen["static"][1]
    assert seen["allocating"][0] == 0 and seen["allocating"][1]
    assert np.array_equal(seen["static"][2], seen["allocating"][2])


def test_shape_that_does_not_split_runs_the_ordinary_kernels():
    check_pair(512, 512, 256, seed=5)


def test_split_that_the_static_array_cannot_hold_is_refused():
    w = runtime.wrappers()
    M, N, K = 640, 640, 4096                    # 100 tiles x 3 chunks x 16 KiB = 4.7 MiB > 4 MiB
    A, B, C = operands(M, N, K, 6, True)
    rc, out = call(w.tiramisu_hip_sgemm_static_scratch, A, B, C, M, N, K, 1.0, 0.0)
    assert rc == 1 and np.array_equal(out, C)
    rc, out = call(w.tiramisu_hip_sgemm, A, B, C, M, N, K, 1.0, 0.0)
    assert rc == 0 and np.array_equal(out, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))
