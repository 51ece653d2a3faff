"""tiramisu_hip_sgemm, the library GEMM behind cublas_gemm() (replaces tiramisu_cublas_sgemm,
tiramisu_cuda_wrappers.cpp:74-115), called through the C ABI on every kernel configuration it
dispatches to: the square tiles chosen for the launch (64, 128, 192, 256), guarded edges, the
64-row split-K configuration with its four prefetch depths, transposed operands, leading
dimensions and offsets.  Small integer data: every sum is exact, comparison for equality with a
float64 product."""
import numpy as np
import pytest

from tiramisu_amd import runtime

pytestmark = pytest.mark.gpu


def run(M, N, K, alpha, beta, tA=False, tB=False, pad=0, off=0, seed=0):
    from gpu_util import DeviceArray
    rng = np.random.RandomState(seed + M + N + K)
    a_rows, a_cols = (K, M) if tA else (M, K)
    b_rows, b_cols = (N, K) if tB else (K, N)
    ldA, ldB, ldC = a_cols + pad, b_cols + pad, N + 2 * pad
    A = rng.randint(-3, 4, a_rows * ldA + off).astype(np.float32)
    B = rng.randint(-3, 4, b_rows * ldB + off + 4).astype(np.float32)
    C = rng.randint(-3, 4, M * ldC + off + 8).astype(np.float32)
    offA, offB, offC = off, off + 4 if off else 0, off + 8 if off else 0
    a = A[offA:offA + a_rows * ldA].reshape(a_rows, ldA)[:, :a_cols].astype(np.float64)
    b = B[offB:offB + b_rows * ldB].reshape(b_rows, ldB)[:, :b_cols].astype(np.float64)
    expected = C.copy()
    c = expected[offC:offC + M * ldC].reshape(M, ldC)[:, :N]
    c[:] = alpha * ((a.T if tA else a) @ (b.T if tB else b)) + (beta * c if beta != 0 else 0)
    dA, dB, dC = DeviceArray(A), DeviceArray(B), DeviceArray(C)
    packed = pad == 0
    runtime.wrappers().tiramisu_hip_sgemm(dA.ptr, dB.ptr, dC.ptr, M, N, K, alpha, beta, 0 if packed else ldA, 0 if packed else ldB,
                                          0 if packed else ldC, offA, offB, offC, tA, tB)
    out = dC.download()
    assert np.array_equal(out, expected)


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (64, 64, 48), (100, 70, 50), (640, 2048, 512), (2048, 2048, 48),
                                   (3072, 3072, 32), (4096, 4096, 64), (33, 17, 9), (8, 8, 4)])
def test_square_tiles(M, N, K):
    run(M, N, K, 1.0, 0.0)
    run(M, N, K, 3.0, 2.0, seed=1)


@pytest.mark.parametrize("K", [256, 384, 512, 1024])
@pytest.mark.parametrize("tB", [False, True])
def test_batch_of_64_rows_splits_k(K, tB):
    # the recurrent product of an LSTM cell (benchmarks/DNN/blocks/LSTM/gpu_lib/generator.cpp:76-84)
    run(64, 2048, K, 1.0, 1.0, tB=tB)
    run(64, 96, K, 2.0, 0.0, tB=tB, seed=2)


@pytest.mark.parametrize("M,N,K", [(256, 256, 8192), (128, 192, 4096), (100, 70, 2500), (640, 640, 4096), (64, 64, 65536)])
@pytest.mark.parametrize("tA,tB", [(False, False), (True, True)])
def test_deep_reductions_split_k_over_workgroups(M, N, K, tA, tB):
    # few 64x64 tiles and K >= 2048: chunks of K on different workgroups, partial tiles through the
    # scratch workspace, the last workgroup of a tile adds them in chunk order
    run(M, N, K, 1.0, 0.0, tA=tA, tB=tB)
    run(M, N, K, 2.0, 1.0, tA=tA, tB=tB, pad=4, off=16, seed=3)


@pytest.mark.parametrize("tA,tB", [(False, True), (True, False), (True, True)])
def test_transposed_operands_padding_and_offsets(tA, tB):
    run(128, 192, 96, 1.0, 1.0, tA=tA, tB=tB)
    run(96, 80, 40, 2.0, 1.0, tA=tA, tB=tB, pad=4, off=12)
    run(64, 2048, 512, 1.0, 1.0, tA=tA, tB=tB, pad=4, off=16)
    run(50, 30, 20, 1.0, 0.0, tA=tA, tB=tB, pad=3, off=5)


def test_seeded_sweep_of_shapes():
    # 80 shapes up to 300 in each dimension, every transposition, with and without padding / offsets
    rng = np.random.RandomState(2026)
    for case in range(80):
        M, N, K = (int(v) for v in rng.randint(1, 301, 3))
        if case % 5 == 0:
            M, N, K = 64 * int(rng.randint(1, 4)), 32 * int(rng.randint(1, 9)), 128 * int(rng.randint(2, 5))
        tA, tB = bool(rng.randint(2)), bool(rng.randint(2))
        pad = int(rng.choice([0, 1, 4]))
        off = int(rng.choice([0, 3, 16]))
        alpha, beta = float(rng.choice([1.0, 2.0, -1.0])), float(rng.choice([0.0, 1.0, 0.5]))
        print("case", case, M, N, K, tA, tB, pad, off, alpha, beta, flush=True)
        run(M, N, K, alpha, beta, tA=tA, tB=tB, pad=pad, off=off, seed=case)


DOUBLE_CASES = [(70, 50, 30, False, False), (64, 96, 128, True, False), (33, 65, 17, False, True), (128, 128, 64, True, True),
                # enough 128 x 128 tiles for the large-tile kernel, ragged in M, N and K, all four transposition cases
                (1500, 1430, 250, False, False), (1500, 1430, 250, True, False), (1500, 1430, 250, False, True), (1411, 1600, 77, True, True),
                (1, 1, 1, False, False), (17, 3000, 5, False, False)]


@pytest.mark.parametrize("M,N,K,tA,tB", DOUBLE_CASES)
def test_double_precision(M, N, K, tA, tB):
    # tiramisu_hip_dgemm (replaces tiramisu_cublas_dgemm, tiramisu_cuda_wrappers.cpp:117-162): fp64 matrix instructions
    from gpu_util import DeviceArray
    rng = np.random.RandomState(M * K)
    A = rng.uniform(-1, 1, (K, M) if tA else (M, K))
    B = rng.uniform(-1, 1, (N, K) if tB else (K, N))
    C = rng.uniform(-1, 1, (M, N))
    expected = 1.5 * ((A.T if tA else A) @ (B.T if tB else B)) + 0.5 * C
    dA, dB, dC = DeviceArray(A), DeviceArray(B), DeviceArray(C)
    runtime.wrappers().tiramisu_hip_dgemm(dA.ptr, dB.ptr, dC.ptr, M, N, K, 1.5, 0.5, 0, 0, 0, 0, 0, 0, tA, tB)
    assert np.max(np.abs(dC.download() - expected)) <= 1e-12 * K
    # integer-valued data: exact, whatever the order of the sums
    A, B, C = np.rint(A * 8), np.rint(B * 8), np.rint(C * 8)
    dA, dB, dC = DeviceArray(A), DeviceArray(B), DeviceArray(C)
    runtime.wrappers().tiramisu_hip_dgemm(dA.ptr, dB.ptr, dC.ptr, M, N, K, 2.0, 0.0, 0, 0, 0, 0, 0, 0, tA, tB)
    assert np.array_equal(dC.download(), 2.0 * ((A.T if tA else A) @ (B.T if tB else B)))


def test_double_precision_leading_dimensions_and_offsets():
    # operands inside larger allocations: leading dimensions wider than the rows, element offsets, beta = 1
    from gpu_util import DeviceArray
    rng = np.random.RandomState(9)
    M, N, K, lda, ldb, ldc, oa, ob, oc = 90, 70, 40, 47, 75, 80, 5, 11, 3
    bufA = np.rint(rng.uniform(-4, 4, oa + M * lda))
    bufB = np.rint(rng.uniform(-4, 4, ob + K * ldb))
    bufC = np.rint(rng.uniform(-4, 4, oc + M * ldc))
    A = bufA[oa:oa + M * lda].reshape(M, lda)[:, :K]
    B = bufB[ob:ob + K * ldb].reshape(K, ldb)[:, :N]
    expected = bufC.copy()
    view = expected[oc:oc + M * ldc].reshape(M, ldc)
    view[:, :N] = -1.0 * (A @ B) + view[:, :N]
    dA, dB, dC = DeviceArray(bufA), DeviceArray(bufB), DeviceArray(bufC)
    runtime.wrappers().tiramisu_hip_dgemm(dA.ptr, dB.ptr, dC.ptr, M, N, K, -1.0, 1.0, lda, ldb, ldc, oa, ob, oc, False, False)
    assert np.array_equal(dC.download(), expected)         # the padding between rows is untouched


def test_freed_device_blocks_are_reused():
    # the runtime keeps freed blocks by size for the next request (generated functions allocate
    # and free their temporaries on every call)
    w = runtime.wrappers()
    a = w.tiramisu_hip_malloc(3 << 20)
    b = w.tiramisu_hip_malloc(3 << 20)
    assert a != b
    w.tiramisu_hip_free(a)
    c = w.tiramisu_hip_malloc(5 << 20)
    d = w.tiramisu_hip_malloc(3 << 20)
    assert d == a and c not in (a, b)
    for p in (b, c, d):
        w.tiramisu_hip_free(p)


def test_deep_reductions_on_two_streams_of_one_thread_use_separate_scratch():
    """One host thread issues deep reductions alternately on two streams without waiting in between: each
    stream has a scratch block of its own (partial tiles and counters would otherwise be shared by launches that
    run at the same time), and every result is the exact integer product."""
    from gpu_util import DeviceArray
    w = runtime.wrappers()
    M, N, K = 128, 192, 8192
    rng = np.random.RandomState(44)
    streams = [w.tiramisu_hip_stream_create(), w.tiramisu_hip_stream_create()]
    jobs = []
    for i in range(6):
        A = rng.randint(-3, 4, (M, K)).astype(np.float32)
        B = rng.randint(-3, 4, (K, N)).astype(np.float32)
        jobs.append((A, B, DeviceArray(A), DeviceArray(B), DeviceArray(np.zeros((M, N), np.float32))))
    blocks = set()
    try:
        for i, (A, B, dA, dB, dC) in enumerate(jobs):
            w.tiramisu_hip_set_stream(streams[i % 2])
            assert w.tiramisu_hip_sgemm(dA.ptr, dB.ptr, dC.ptr, M, N, K, 1.0, 0.0, 0, 0, 0, 0, 0, 0, False, False) == 0
            blocks.add((i % 2, w.tiramisu_hip_sgemm_workspace()))
        for s in streams:
            w.tiramisu_hip_set_stream(s)
            w.tiramisu_hip_stream_synchronize(0)
    finally:
        w.tiramisu_hip_set_stream(None)
    assert len(blocks) == 2 and len({b for _, b in blocks}) == 2 and all(b for _, b in blocks)
    for A, B, dA, dB, dC in jobs:
        assert np.array_equal(dC.download(), (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))
        for d in (dA, dB, dC):
            d.free()
    for s in streams:
        w.tiramisu_hip_stream_destroy(s)


def test_calls_gathered_in_a_batch_scope_give_the_results_of_separate_calls():
    """tiramisu_hip_batch_begin / _end: four recurrent-cell products of one shape (one launch, a problem per
    blockIdx.z), then a product of another shape and one that takes the element-per-thread kernel (launched one by
    one), all exact on small integers; nothing is written before _end."""
    from gpu_util import DeviceArray
    w = runtime.wrappers()
    rng = np.random.RandomState(45)
    shapes = [(64, 2048, 512)] * 4 + [(640, 256, 128), (16, 16, 4)]
    jobs = []
    for M, N, K in shapes:
        A = rng.randint(-3, 4, (M, K)).astype(np.float32)
        B = rng.randint(-3, 4, (K, N)).astype(np.float32)
        C = rng.randint(-3, 4, (M, N)).astype(np.float32)
        jobs.append((A, B, C, DeviceArray(A), DeviceArray(B), DeviceArray(C)))
    assert w.tiramisu_hip_batch_end() == 1                     # no scope open
    assert w.tiramisu_hip_batch_begin() == 0
    assert w.tiramisu_hip_batch_begin() == 1                   # scopes do not nest
    for (M, N, K), (A, B, C, dA, dB, dC) in zip(shapes, jobs):
        assert w.tiramisu_hip_sgemm(dA.ptr, dB.ptr, dC.ptr, M, N, K, 1.0, 1.0, 0, 0, 0, 0, 0, 0, False, False) == 0
    assert np.array_equal(jobs[0][5].download(), jobs[0][2])   # gathered, not launched
    assert w.tiramisu_hip_batch_end() == 0
    for A, B, C, dA, dB, dC in jobs:
        assert np.array_equal(dC.download(), (A.astype(np.float64) @ B.astype(np.float64) + C).astype(np.float32))
        for d in (dA, dB, dC):
            d.free()
