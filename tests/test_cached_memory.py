"""Memory the runtime keeps between calls (include/tiramisu_hip_wrappers.h: tiramisu_hip_kept_scratch,
tiramisu_hip_release_cached_memory, tiramisu_hip_cached_memory_bytes; the reference's generated code allocates and
frees everything on every call, tiramisu_cuda_wrappers.cpp:55-68, and keeps nothing): the third plane of a
time-tiled stencil, the workspaces of deep GEMM reductions and the idle blocks of the pool are counted, can be given
back to HIP in one call, and come back at the next call that needs them -- with the same results."""
import ctypes
import os

import numpy as np
import pytest

from oracle import reference_loops as ref
from tiramisu_amd import runtime

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")


def heat2d_on_gpu(n, steps, planes):
    w = runtime.wrappers()
    dev = w.tiramisu_hip_malloc(planes.nbytes)
    w.tiramisu_hip_memcpy_to_device(dev, planes.ctypes.data, planes.nbytes)
    name = "heat2d_%dx%d" % (n, steps)
    runtime.load(PROGRAMS, name)(runtime.Buffer.from_device(dev, planes.shape, np.float32))
    w.tiramisu_hip_stream_synchronize(0)
    out = np.empty_like(planes)
    w.tiramisu_hip_memcpy_to_host(out.ctypes.data, dev, planes.nbytes)
    w.tiramisu_hip_free(dev)
    return out


def deep_gemm(seed):
    from gpu_util import DeviceArray
    w = runtime.wrappers()
    M, N, K = 128, 192, 8192
    rng = np.random.RandomState(seed)
    A = rng.randint(-3, 4, (M, K)).astype(np.float32)
    B = rng.randint(-3, 4, (K, N)).astype(np.float32)
    dA, dB, dC = DeviceArray(A), DeviceArray(B), DeviceArray(np.zeros((M, N), np.float32))
    assert w.tiramisu_hip_sgemm(dA.ptr, dB.ptr, dC.ptr, M, N, K, 1.0, 0.0, 0, 0, 0, 0, 0, 0, False, False) == 0
    out = dC.download()
    for d in (dA, dB, dC):
        d.free()
    assert np.array_equal(out, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))


def test_kept_scratch_is_one_block_per_site_and_grows_on_demand():
    w = runtime.wrappers()
    w.tiramisu_hip_release_cached_memory()
    site_a, site_b = ctypes.c_char(), ctypes.c_char()
    fresh = ctypes.c_int32(-1)
    a = w.tiramisu_hip_kept_scratch(ctypes.addressof(site_a), 1 << 20, ctypes.byref(fresh))
    assert a and fresh.value == 1
    assert w.tiramisu_hip_kept_scratch(ctypes.addressof(site_a), 1 << 20, ctypes.byref(fresh)) == a and fresh.value == 0
    assert w.tiramisu_hip_kept_scratch(ctypes.addressof(site_a), 1 << 10, None) == a         # a smaller request: the same block
    b = w.tiramisu_hip_kept_scratch(ctypes.addressof(site_b), 1 << 20, ctypes.byref(fresh))
    assert b and b != a and fresh.value == 1
    assert w.tiramisu_hip_cached_memory_bytes() == 2 << 20
    w.tiramisu_hip_kept_scratch(ctypes.addressof(site_a), 3 << 20, ctypes.byref(fresh))       # grows: a new block
    assert fresh.value == 1
    assert w.tiramisu_hip_cached_memory_bytes() == 4 << 20
    # another stream of the same thread has blocks of its own
    s = w.tiramisu_hip_stream_create()
    w.tiramisu_hip_set_stream(s)
    try:
        c = w.tiramisu_hip_kept_scratch(ctypes.addressof(site_b), 1 << 20, ctypes.byref(fresh))
        assert c and c != b and fresh.value == 1
    finally:
        w.tiramisu_hip_set_stream(None)
        w.tiramisu_hip_stream_destroy(s)
    assert w.tiramisu_hip_release_cached_memory() == 5 << 20
    assert w.tiramisu_hip_cached_memory_bytes() == 0


def test_release_gives_back_the_third_plane_workspaces_and_idle_blocks():
    w = runtime.wrappers()
    w.tiramisu_hip_release_cached_memory()
    assert w.tiramisu_hip_cached_memory_bytes() == 0
    n, steps = 1030, 9                                    # three launches through a third plane of n x n floats
    rng = np.random.RandomState(11)
    planes = rng.uniform(0, 1, (2, n, n)).astype(np.float32)
    expected = ref.heat2d(planes[0], steps, boundary_other=planes[1])
    print("heat2d", n, steps, flush=True)
    assert np.array_equal(heat2d_on_gpu(n, steps, planes.copy()), expected)
    plane, both = n * n * 4, 2 * n * n * 4
    # kept: the third plane; idle in the pool: the block that held the two planes
    assert w.tiramisu_hip_cached_memory_bytes() == plane + both
    print("deep gemm", flush=True)
    deep_gemm(3)
    assert w.tiramisu_hip_sgemm_workspace()
    held = w.tiramisu_hip_cached_memory_bytes()
    assert held > plane + both
    assert w.tiramisu_hip_release_cached_memory() == held
    assert w.tiramisu_hip_cached_memory_bytes() == 0
    assert not w.tiramisu_hip_sgemm_workspace()
    # everything comes back at the next call that needs it
    print("heat2d and deep gemm after the release", flush=True)
    assert np.array_equal(heat2d_on_gpu(n, steps, planes.copy()), expected)
    deep_gemm(4)
    assert w.tiramisu_hip_cached_memory_bytes() == held
