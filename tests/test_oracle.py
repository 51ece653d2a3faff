"""CPU-side tests (no GPU): the CPU back-end restatement against the numpy restatements of the
reference's wrapper loops, and the schedule algebra against brute-force enumeration."""
import itertools
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from oracle import reference_loops as ref
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tests", "programs")


def cpu_program(name, directory=PROGRAMS):
    return runtime.Program(oracle_build.cpu_program_library(directory, name), name, needs_gpu_runtime=False)


def ints(rng, shape):
    return (rng.randint(0, 10, shape) - 5).astype(np.float32)


# ---------------------------------------------------------------- oracle pins

def test_gemm_restatement_closed_forms():
    # all-ones: C = alpha*K + beta (reference: sgemm/cpu/sgemm_wrapper.cpp:166-169)
    M, N, K = 5, 7, 9
    A, B, C = np.ones((M, K), np.float32), np.ones((K, N), np.float32), np.ones((M, N), np.float32)
    assert np.array_equal(ref.sgemm(A, B, C, 3.0, 2.0), np.full((M, N), 3.0 * K + 2.0, np.float32))
    # a transposed operand or a dropped accumulation term must fail this: compare with float64 matmul
    rng = np.random.RandomState(1)
    A, B, C = ints(rng, (M, K)), ints(rng, (K, N)), ints(rng, (M, N))
    assert np.array_equal(ref.gemm_accumulate(A, B, C), (C.astype(np.float64) + A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))
    assert np.array_equal(ref.sgemm(A, B, C, 0.0, 1.0), C)
    assert np.array_equal(ref.sgemm(A, B, C, 1.0, 0.0), (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))


def test_strided_gemm_restatement_against_numpy_slicing():
    """sgemm_strided (leading dimensions, element offsets, transposition as tiramisu_cublas_sgemm defines
    them, tiramisu_cuda_wrappers.cpp:74-115) against plain numpy: the operands are cut out of larger flat
    buffers by slicing and .T, so a swapped ld / offset / transposition rule fails.  Integer data: exact."""
    rng = np.random.RandomState(74)
    M, N, K = 5, 7, 6
    for tA in (False, True):
        for tB in (False, True):
            ldA, ldB, ldC = (M + 3 if tA else K + 2), (K + 1 if tB else N + 4), N + 5
            offA, offB, offC = 3, 11, 2
            rowsA, rowsB = (K if tA else M), (N if tB else K)
            Abuf, Bbuf = ints(rng, (offA + rowsA * ldA,)), ints(rng, (offB + rowsB * ldB,))
            Cbuf = ints(rng, (offC + M * ldC,))
            A2 = Abuf[offA:offA + rowsA * ldA].reshape(rowsA, ldA)[:, :(M if tA else K)]
            B2 = Bbuf[offB:offB + rowsB * ldB].reshape(rowsB, ldB)[:, :(K if tB else N)]
            opA, opB = (A2.T if tA else A2), (B2.T if tB else B2)
            expected = Cbuf.copy()
            Cview = expected[offC:offC + M * ldC].reshape(M, ldC)[:, :N]
            Cview[...] = (3.0 * (opA.astype(np.float64) @ opB.astype(np.float64)) + 2.0 * Cview).astype(np.float32)
            out = ref.sgemm_strided(Abuf, Bbuf, Cbuf, M, N, K, 3.0, 2.0, ldA, ldB, ldC, offA, offB, offC, tA, tB)
            assert np.array_equal(out, expected), (tA, tB)
    # ld == 0 means tightly packed; beta == 0 ignores what C held (NaN included)
    A, B = ints(rng, (M, K)), ints(rng, (K, N))
    C = np.full((M, N), np.nan, np.float32)
    out = ref.sgemm_strided(A, B, C, M, N, K, 1.0, 0.0, 0, 0, 0, 0, 0, 0, False, False)
    assert np.array_equal(out, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))
    out = ref.sgemm_strided(A.T.copy(), B.T.copy(), C, M, N, K, 1.0, 0.0, 0, 0, 0, 0, 0, 0, True, True)
    assert np.array_equal(out, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))


# ---------------------------------------------------------------- CPU back-end vs restatements

def test_cpu_gemm_gpu_tile():
    rng = np.random.RandomState(167)
    A, B, C = ints(rng, (96, 64)), ints(rng, (64, 160)), ints(rng, (96, 160))
    expected = ref.gemm_accumulate(A, B, C)
    cpu_program("gemm_gpu_tile")(A, B, C)
    assert np.array_equal(C, expected)


def test_cpu_transpose():
    rng = np.random.RandomState(168)
    A = ints(rng, (144, 80))
    out = np.zeros((80, 144), np.float32)
    cpu_program("transpose_gpu_tile")(A, out)
    assert np.array_equal(out, ref.transpose(A))


def test_cpu_gemm_register_tile():
    rng = np.random.RandomState(170)
    A, B, C = ints(rng, (96, 100)), ints(rng, (100, 180)), ints(rng, (96, 180))
    expected = ref.gemm_accumulate(A, B, C)
    cpu_program("gemm_register_tile")(A, B, C)
    assert np.array_equal(C, expected)


def test_row_filter_restatement_pins():
    # a single unit tap is a shifted copy; all-ones taps on all-ones pixels count the taps
    img = ints(np.random.RandomState(3), (6, 12))
    for t in range(5):
        taps = np.zeros(5, np.float32)
        taps[t] = 1.0
        assert np.array_equal(ref.row_filter(img, taps), img[:, t:t + 8])
    assert np.all(ref.row_filter(np.ones((4, 9), np.float32), np.ones(5, np.float32)) == 5.0)
    # against plain loops
    taps = ints(np.random.RandomState(4), (5,))
    loops = np.zeros((6, 8), np.float32)
    for r in range(6):
        for c in range(8):
            loops[r, c] = sum(float(img[r, c + t]) * float(taps[t]) for t in range(5))
    assert np.array_equal(ref.row_filter(img, taps), loops)


def test_resample_restatement_pins():
    # a constant image resamples to itself; an image linear in x and y is reproduced exactly where
    # no neighbour is clamped (bilinear interpolation is exact on such images)
    assert np.all(ref.resample_bilinear(np.full((20, 30), 7, np.uint8)) == 7.0)
    h, w = 40, 48
    yy, xx = np.mgrid[0:h, 0:w]
    img = (2 * yy + xx).astype(np.uint8)
    out = ref.resample_bilinear(img)
    fy = yy * 0.96875 + xx * 0.0625 - 1.5
    fx = xx * 0.96875 - yy * 0.0625 + 2.25
    inside = (fy >= 0) & (fy <= h - 2) & (fx >= 0) & (fx <= w - 2)
    assert inside.sum() > 1000
    assert np.array_equal(out[inside], (2 * fy + fx)[inside].astype(np.float32))


def test_cpu_resample_bilinear():
    src = np.random.RandomState(77).randint(0, 256, (90, 132)).astype(np.uint8)
    out = np.zeros((90, 132), np.float32)
    cpu_program("resample_bilinear")(src, out)
    assert np.array_equal(out, ref.resample_bilinear(src))


def test_cpu_taps_in_constant_memory():
    rng = np.random.RandomState(61)
    img, taps = ints(rng, (70, 100)), ints(rng, (5,))
    out = np.zeros((70, 96), np.float32)
    cpu_program("taps_in_constant_memory")(img, taps, out)
    assert np.array_equal(out, ref.row_filter(img, taps))


def test_cpu_alloc_in_time_loop():
    P = np.zeros((3, 24, 24), np.int32)
    Q = np.zeros((3, 40, 40), np.int32)
    cpu_program("alloc_in_time_loop")(P, Q)
    eP, eQ = ref.alloc_in_time_loop_expected(3, 24, 40)
    assert np.array_equal(P, eP) and np.array_equal(Q, eQ)


# ---------------------------------------------------------------- schedule algebra, brute force

P_, Q_ = 10, 14


def stamps(name):
    clock = np.zeros(1, np.int32)
    stamp = np.full((P_, Q_), -1, np.int32)
    cpu_program(name)(clock, stamp)
    assert clock[0] == P_ * Q_
    return stamp


def order_to_stamps(points):
    out = np.full((P_, Q_), -1, np.int32)
    for n, (i, j) in enumerate(points):
        out[i, j] = n
    return out


def all_points():
    return list(itertools.product(range(P_), range(Q_)))


def test_order_identity():
    assert np.array_equal(stamps("order_identity"), order_to_stamps(all_points()))


def test_order_split():
    pts = sorted(all_points(), key=lambda p: (p[0], p[1] // 4, p[1] % 4))
    assert np.array_equal(stamps("order_split"), order_to_stamps(pts))


def test_order_tile():
    pts = sorted(all_points(), key=lambda p: (p[0] // 3, p[1] // 5, p[0] % 3, p[1] % 5))
    assert np.array_equal(stamps("order_tile"), order_to_stamps(pts))


def test_order_interchange():
    pts = sorted(all_points(), key=lambda p: (p[1], p[0]))
    assert np.array_equal(stamps("order_interchange"), order_to_stamps(pts))


def test_order_skew_shift():
    pts = sorted(all_points(), key=lambda p: (p[0], 2 * p[0] + p[1] + 3))
    assert np.array_equal(stamps("order_skew_shift"), order_to_stamps(pts))


def test_order_fuse_outer():
    # per row: Q stamps read the clock before any tick of that row runs
    expected = np.repeat(np.arange(P_, dtype=np.int32)[:, None] * Q_, Q_, axis=1)
    assert np.array_equal(stamps("order_fuse_outer"), expected)


def test_order_tags_do_not_change_results():
    pts = sorted(all_points(), key=lambda p: (p[0], p[1] // 4, p[1] % 4))
    assert np.array_equal(stamps("order_tags"), order_to_stamps(pts))
