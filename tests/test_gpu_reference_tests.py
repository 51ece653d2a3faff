"""GPU parity tests for the schedule-faithful (generic) emitter: programs with the features of
the reference's own GPU tests (tests/test_162.cpp, test_164-171.cpp, test_197.cpp of the
reference tree), compiled by the HIP back-end, called through the C ABI and compared

  * with the nested-loop references the reference's wrappers use (numpy restatements), and
  * with the CPU-generated code of the very same Tiramisu program (CPU back-end restatement).

Inputs are small integers, as in the reference's wrappers, so fp32 results are exact and every
comparison is bit-for-bit."""
import os
import re

import numpy as np
import pytest

from oracle import build as oracle_build
from oracle import reference_loops as ref
from tiramisu_amd import runtime

pytestmark = pytest.mark.gpu


def ints(rng, shape):
    return (rng.randint(0, 10, shape) - 5).astype(np.float32)


def cpu_variant(programs_dir, name):
    return runtime.Program(oracle_build.cpu_program_library(programs_dir, name), name, needs_gpu_runtime=False)


def test_gemm_gpu_tile(programs_dir):
    rng = np.random.RandomState(167)
    A, B, C = ints(rng, (96, 64)), ints(rng, (64, 160)), ints(rng, (96, 160))
    expected = ref.gemm_accumulate(A, B, C)
    C_cpu = C.copy()
    cpu_variant(programs_dir, "gemm_gpu_tile")(A, B, C_cpu)
    runtime.load(programs_dir, "gemm_gpu_tile")(A, B, C)
    assert np.array_equal(C, expected)
    assert np.array_equal(C, C_cpu)


def test_transpose_gpu_tile(programs_dir):
    rng = np.random.RandomState(168)
    A = ints(rng, (144, 80))
    out = np.zeros((80, 144), np.float32)
    runtime.load(programs_dir, "transpose_gpu_tile")(A, out)
    assert np.array_equal(out, ref.transpose(A))


def test_gemm_register_tile(programs_dir):
    rng = np.random.RandomState(170)
    A, B, C = ints(rng, (96, 100)), ints(rng, (100, 180)), ints(rng, (96, 180))
    expected = ref.gemm_accumulate(A, B, C)
    C_cpu = C.copy()
    cpu_variant(programs_dir, "gemm_register_tile")(A, B, C_cpu)
    runtime.load(programs_dir, "gemm_register_tile")(A, B, C)
    assert np.array_equal(C, expected)
    assert np.array_equal(C, C_cpu)


def test_taps_in_constant_memory_with_automatic_copies(programs_dir):
    # host buffers in, host buffer out: every copy (one of them to a constant-memory symbol) is
    # inserted by codegen() from the CPU/GPU buffer mapping
    rng = np.random.RandomState(61)
    img, taps = ints(rng, (70, 100)), ints(rng, (5,))
    out = np.full((70, 96), -1.0, np.float32)
    out_cpu = out.copy()
    cpu_variant(programs_dir, "taps_in_constant_memory")(img, taps, out_cpu)
    prog = runtime.load(programs_dir, "taps_in_constant_memory")
    prog(img, taps, out)
    assert np.array_equal(out, ref.row_filter(img, taps))
    assert np.array_equal(out, out_cpu)
    # the symbol keeps no state between calls: new taps, new result
    taps2 = ints(np.random.RandomState(62), (5,))
    prog(img, taps2, out)
    assert np.array_equal(out, ref.row_filter(img, taps2))


@pytest.mark.parametrize("M,N,K", [
    (100, 70, 50),     # ragged in every direction, rows not 16-byte aligned
    (64, 64, 64),      # whole tiles
    (1, 1, 1),
    (130, 33, 7),      # K smaller than a slice
    (257, 129, 65),
    (0, 5, 5), (5, 0, 5),   # empty iteration spaces: nothing is launched, C untouched
    (5, 5, 0),         # empty reduction: C = beta * C
])
@pytest.mark.parametrize("name", ["sgemm_runtime_sizes", "sgemm_runtime_sizes_generic"])
def test_sgemm_runtime_sizes(programs_dir, name, M, N, K):
    # one compiled function, sizes read from a buffer at run time; once through the contraction
    # emitter and once through the schedule-faithful emitter
    from gpu_util import DeviceArray
    rng = np.random.RandomState(1000 + M + N + K)
    A, B, C = ints(rng, (M, K)), ints(rng, (K, N)), ints(rng, (M, N))
    sizes = np.array([M, N, K], np.int32)
    scal = np.array([2.0, -1.0], np.float32)
    expected = ref.sgemm(A, B, C, 2.0, -1.0)
    C_cpu = C.copy()
    cpu_variant(programs_dir, name)(sizes, scal, A, B, C_cpu)
    assert np.array_equal(C_cpu, expected)
    # device buffers carry a few extra elements so that empty matrices still have an address
    dA, dB, dC = (DeviceArray(np.concatenate([x.ravel(), np.zeros(4, np.float32)])) for x in (A, B, C))
    prog = runtime.load(programs_dir, name)
    w = runtime.wrappers()
    prog(sizes, scal, runtime.Buffer.from_device(dA.ptr, (M, K), np.float32),
         runtime.Buffer.from_device(dB.ptr, (K, N), np.float32), runtime.Buffer.from_device(dC.ptr, (M, N), np.float32))
    w.tiramisu_hip_stream_synchronize(0)
    out = dC.download()[:M * N].reshape(M, N)
    assert np.array_equal(out, expected)


def test_resample_bilinear_scheduled_constants(programs_dir):
    # constants declared at a loop level (scalars in the kernel), clamped data-dependent indices
    from gpu_util import DeviceArray
    src = np.random.RandomState(77).randint(0, 256, (90, 132)).astype(np.uint8)
    d_src, d_dst = DeviceArray(src), DeviceArray(np.zeros((90, 132), np.float32))
    runtime.load(programs_dir, "resample_bilinear")(d_src.buffer(), d_dst.buffer())
    out = d_dst.download()
    out_cpu = np.zeros((90, 132), np.float32)
    cpu_variant(programs_dir, "resample_bilinear")(src, out_cpu)
    # every intermediate value is exactly representable (weights are multiples of 1/32), so
    # the comparison is bit for bit whatever the contraction of multiply-adds
    assert np.array_equal(out, ref.resample_bilinear(src))
    assert np.array_equal(out, out_cpu)


def test_low_level_api_three_dimensional_gpu_tile(programs_dir):
    # explicit function object, isl-string domain and access, hand-driven pipeline, 3-D gpu_tile
    from gpu_util import DeviceArray
    d = DeviceArray(np.full((10, 10), -1, np.int32))
    runtime.load(programs_dir, "low_level_api")(d.buffer())
    i, k = np.mgrid[0:10, 0:10]
    assert np.array_equal(d.download(), (100 * i + k + 7).astype(np.int32))


def test_alloc_in_time_loop(programs_dir):
    P = np.zeros((3, 24, 24), np.int32)
    Q = np.zeros((3, 40, 40), np.int32)
    runtime.load(programs_dir, "alloc_in_time_loop")(P, Q)
    eP, eQ = ref.alloc_in_time_loop_expected(3, 24, 40)
    assert np.array_equal(P, eP) and np.array_equal(Q, eQ)


@pytest.mark.parametrize("M,N,K,alpha,beta,pad,off", [
    (1, 2, 3, 1.0, 0.0, 0, 0),        # the reference's smallest case (test_162: 1x2x3)
    (12, 20, 7, 3.0, 2.0, 0, 0),
    (33, 40, 9, 0.0, 1.0, 3, 5),      # alpha = 0 keeps beta*C
    (64, 96, 32, 2.0, 0.0, 4, 8),     # beta = 0 must not read C
    (130, 70, 50, -1.0, 0.5, 1, 3),   # MFMA path with ragged edges and unaligned rows
    (256, 256, 64, 1.0, 1.0, 0, 0),   # MFMA path, whole tiles
])
@pytest.mark.parametrize("name,real", [("sgemm_library_call", np.float32), ("dgemm_library_call", np.float64)])
def test_sgemm_library_call(programs_dir, name, real, M, N, K, alpha, beta, pad, off):
    rng = np.random.RandomState(162 + M)
    ldA, ldB, ldC = M + pad, N + pad, N + 2 * pad
    sizes = np.array([M, N, K, ldA, ldB, ldC, off, off + 1, off + 2], np.int32)
    scal = np.array([alpha, beta], real)
    A = ints(rng, (K + 1, ldA)).astype(real)     # stored transposed: K rows
    B = ints(rng, (K + 1, ldB)).astype(real)
    C = ints(rng, (M + 1, ldC)).astype(real)
    if beta == 0.0:
        C[:] = np.nan               # reading C would poison the result
    expected = ref.sgemm_strided(A, B, C, M, N, K, alpha, beta, ldA, ldB, ldC, off, off + 1, off + 2, True, False)
    runtime.load(programs_dir, name)(sizes, scal, A, B, C)
    assert np.array_equal(C, expected, equal_nan=True)


@pytest.mark.parametrize("name,kind", [("sgemm_shared_regs", "mfma-contraction"), ("sgemm_shared_regs_generic", "generic")])
def test_sgemm_cache_shared_register_tile(programs_dir, name, kind):
    # generator3-style staged sgemm: LDS tiles via cache_shared, 4x2 register tile, alpha/beta;
    # once through the MFMA kernel (tiles and register tile proven sound), once as scheduled
    assert re.search(r"^// _kernel_\d+: " + kind, open(os.path.join(programs_dir, "build", name + ".o.hip")).read(), re.M)
    rng = np.random.RandomState(3)
    M, N, K = 256, 192, 64
    A, B, C = ints(rng, (M, K)), ints(rng, (K, N)), ints(rng, (M, N))
    scal = np.array([3.0, 2.0], np.float32)
    expected = ref.sgemm(A, B, C, 3.0, 2.0)
    runtime.load(programs_dir, name)(scal, A, B, C)
    assert np.array_equal(C, expected)


def test_gemm_uint8_cache_shared(programs_dir):
    # uint8 arithmetic wraps modulo 256 (reference: tutorials/developers/tutorial_04gpu2 wrapper)
    rng = np.random.RandomState(4)
    S = 128
    A = rng.randint(0, 256, (S, S)).astype(np.uint8)
    B = rng.randint(0, 256, (S, S)).astype(np.uint8)
    C = rng.randint(0, 256, (S, S)).astype(np.uint8)
    expected = ((C.astype(np.int64) + A.astype(np.int64) @ B.astype(np.int64)) % 256).astype(np.uint8)
    runtime.load(programs_dir, "gemm_u8_shared")(A, B, C)
    assert np.array_equal(C, expected)


@pytest.mark.parametrize("tag,tA,tB,pad,origin", [("nn", False, False, 0, 0), ("nt", False, True, 0, 0), ("tn", True, False, 0, 0),
                                                  ("tt", True, True, 0, 0), ("pitched", False, True, 3, 2)])
def test_gemm_operand_layouts(programs_dir, tag, tA, tB, pad, origin):
    # tests/programs/gemm_operand_layouts.cpp: every storage order of the two operands, and operands
    # inside larger buffers (pitch and origin not multiples of 4 elements), through the MFMA emitter
    from gpu_util import DeviceArray
    M, N, K = 96, 80, 72
    rng = np.random.RandomState(len(tag) + 7 * pad)
    a_rows, a_cols = (K, M) if tA else (M, K)
    b_rows, b_cols = (N, K) if tB else (K, N)
    bufA, bufB = ints(rng, (a_rows + origin, a_cols + pad)), ints(rng, (b_rows + origin, b_cols + pad))
    C = ints(rng, (M, N))
    shift = 1 if pad else 0
    a = bufA[origin:origin + a_rows, shift:shift + a_cols]
    b = bufB[origin:origin + b_rows, shift:shift + b_cols]
    expected = ref.gemm_accumulate(np.ascontiguousarray(a.T if tA else a), np.ascontiguousarray(b.T if tB else b), C)
    assert re.search(r"^// _kernel_\d+: mfma-contraction", open(os.path.join(programs_dir, "build", "gemm_layout_%s.o.hip" % tag)).read(), re.M)
    C_cpu = C.copy()
    cpu_variant(programs_dir, "gemm_layout_" + tag)(bufA, bufB, C_cpu)
    dA, dB, dC = DeviceArray(bufA), DeviceArray(bufB), DeviceArray(C)
    runtime.load(programs_dir, "gemm_layout_" + tag)(dA.buffer(), dB.buffer(), dC.buffer())
    out = dC.download()
    assert np.array_equal(out, expected) and np.array_equal(out, C_cpu)


def test_gemm_two_products_with_batch(programs_dir):
    # tests/programs/gemm_two_products.cpp: two products per reduction step, batch on a third block
    # index (flattened with the rows into M), bias as fused initialisation
    from gpu_util import DeviceArray
    NB, M, N, K = 3, 64, 96, 80
    rng = np.random.RandomState(380)
    W, R = ints(rng, (N, K)), ints(rng, (N, K))
    x, h = ints(rng, (NB, M, K)), ints(rng, (NB, M, K))
    bias = ints(rng, (N,))
    expected = (bias[None, None, :].astype(np.float64) + x.astype(np.float64) @ W.T.astype(np.float64) +
                h.astype(np.float64) @ R.T.astype(np.float64)).astype(np.float32)
    text = open(os.path.join(programs_dir, "build", "gemm_two_products.o.hip")).read()
    assert "2 product term(s), fused initialisation" in text
    out_cpu = np.zeros((NB, M, N), np.float32)
    cpu_variant(programs_dir, "gemm_two_products")(W, R, x, h, bias, out_cpu)
    devs = [DeviceArray(a) for a in (W, R, x, h, bias, np.full((NB, M, N), -1, np.float32))]
    runtime.load(programs_dir, "gemm_two_products")(*[d.buffer() for d in devs])
    out = devs[-1].download()
    assert np.array_equal(out, expected) and np.array_equal(out_cpu, expected)
