"""GPU generator programs of the reference tree, compiled unchanged by this build
(tests/reference_programs/build_reference_programs.py) and run through their generated functions'
C ABI with host buffers, compared with numpy restatements of what the programs' text computes
(oracle/reference_loops.py: ref_*_gpu).  The programs copy to and from the GPU themselves."""
import ctypes
import os

import numpy as np
import pytest

from oracle import reference_loops as ref
from tiramisu_amd import runtime

HERE = os.path.dirname(os.path.abspath(__file__))


def library(name):
    return os.path.join(HERE, "reference_programs", "build", "lib%s.so" % name)


PROGRAMS = {"cvtcolorgpu": "cvtcolorgpu_tiramisu", "gaussiangpu": "gaussiangpu_tiramisu", "heat2dgpu": "heat2dgpu_tiramisu",
            "convolutiongpu": "convolutiongpu_tiramisu", "fusiongpu": "fusiongpu_tiramisu",
            "rgbyuv420gpu": "rgbyuv420gpu_tiramisu", "warp_affinegpu": "warp_affinegpu_tiramisu", "edgegpu": "edge_tiramisu"}


def test_restatements_on_closed_forms():
    # gray of a gray pixel is itself (the three weights sum to 2^14); binomial blur of a constant
    # image is the constant; the heat sweep of a constant interior gives 0.3 + 4*0.4 = 1.9 times it
    rgb = np.stack([np.full((4, 5), v, np.uint8) for v in (200, 200, 200)])
    assert np.all(ref.ref_cvtcolor_gpu(rgb) == 200)
    k = np.array([1, 4, 6, 4, 1], np.float32)
    assert np.all(ref.ref_gaussian_gpu(np.full((2, 12, 14), 37, np.uint8), k, k / 256) == 37)
    g = np.ones((8, 8), np.float32)
    out = ref.ref_heat2d_gpu(g)
    assert np.all(out[1:-1, 1:-1] == np.float32(1.0) * np.float32(0.3) + np.float32(4.0) * np.float32(0.4))
    assert np.all(out[0] == 0) and np.all(out[:, -1] == 0)
    # identity filter; (255 - x) + 2x = 255 + x; gray pixels: y = (220 v + 128) % 256 + 16 and, the chroma
    # weights cancelling, u = v = 128 % 256 + 128 = 256, which is 0 as uint8; a constant image warps to itself; the edge filter of a constant is 0
    img = np.random.RandomState(2).randint(0, 256, (3, 12, 14)).astype(np.uint8)
    ident = np.zeros((3, 3), np.float32)
    ident[1, 1] = 1
    assert np.array_equal(ref.ref_convolution_gpu(img, ident), img[:, 1:-1, 1:-1])
    f, g2, h, k2 = ref.ref_fusion_gpu(img)
    assert np.array_equal(h, (img.astype(np.int32) + 255).astype(np.uint8)) and np.array_equal(f, 255 - img)
    gray = np.stack([img[0]] * 3)
    y, u, v = ref.ref_rgbyuv420_gpu(gray)
    assert np.array_equal(y, ((220 * gray[0].astype(np.int32) + 128) % 256 + 16).astype(np.uint8))
    assert np.all(u == 0) and np.all(v == 0)
    assert np.allclose(ref.ref_warp_affine_gpu(np.full((20, 24), 77, np.uint8)), 77.0, rtol=1e-6)
    assert np.all(ref.ref_edge_gpu(np.full((3, 12, 14), 200, np.uint8)) == 0)
    # edge, element by element in uint8 scalars (sums wrap before the division, as in Halide)
    small = np.random.RandomState(9).randint(0, 256, (1, 7, 8)).astype(np.uint8)
    with np.errstate(over="ignore"):
        u8 = lambda j, i: small[0, j, i]
        ring = lambda j, i: (u8(j, i) + u8(j + 1, i) + u8(j + 2, i) + u8(j, i + 1) + u8(j + 2, i + 1) + u8(j, i + 2) + u8(j + 1, i + 2)
                             + u8(j + 2, i + 2)) // np.uint8(8)
        by_hand = np.array([[(ring(j + 1, i + 1) - ring(j, i + 2)) + (ring(j + 1, i + 2) - ring(j, i + 1)) for i in range(4)] for j in range(3)],
                           np.uint8)
    assert np.array_equal(ref.ref_edge_gpu(small)[0], by_hand)
    assert int(ring(0, 0)) == (sum(int(small[0, j, i]) for j in range(3) for i in range(3)) - int(small[0, 1, 1])) % 256 // 8


@pytest.mark.parametrize("name", sorted(PROGRAMS))
def test_generated_library_exports_its_function(name):
    if not os.path.exists(library(name)):
        pytest.skip("reference tree was absent when the libraries were built")
    runtime.wrappers()
    assert hasattr(ctypes.CDLL(library(name)), PROGRAMS[name])


def load(name):
    if not os.path.exists(library(name)):
        pytest.skip("reference tree was absent when the libraries were built")
    return runtime.Program(library(name), PROGRAMS[name])


@pytest.mark.gpu
@pytest.mark.parametrize("M,N", [(48, 64), (37, 53), (1, 70), (70, 1), (129, 257)])   # whole tiles, ragged, a single row / column
def test_reference_cvtcolorgpu(M, N):
    rgb = np.random.RandomState(M).randint(0, 256, (3, M, N)).astype(np.uint8)
    out = np.zeros((M, N), np.uint8)
    load("cvtcolorgpu")(np.array([N, M], np.int32), rgb, out)
    assert np.array_equal(out, ref.ref_cvtcolor_gpu(rgb))


@pytest.mark.gpu
@pytest.mark.parametrize("C,M,N", [(3, 69, 101), (1, 37, 37)])
def test_reference_gaussiangpu(C, M, N):
    # the wrapper's own taps (benchmarks/halide/wrapper_gaussiangpu.cpp:39-40): every value stays exact
    kx = np.array([1, 4, 6, 4, 1], np.float32)
    ky = kx / np.float32(256)
    img = np.random.RandomState(N).randint(0, 256, (C, M, N)).astype(np.uint8)
    out = np.zeros((C, M - 5, N - 5), np.uint8)
    load("gaussiangpu")(np.array([N, M, C], np.int32), img, kx, ky, out)
    assert np.array_equal(out, ref.ref_gaussian_gpu(img, kx, ky))


@pytest.mark.gpu
@pytest.mark.parametrize("n", [62, 92, 47])
def test_reference_heat2dgpu(n):
    grid = np.random.RandomState(n).uniform(0, 1, (n, n)).astype(np.float32)
    out = np.full((n, n), -1.0, np.float32)
    load("heat2dgpu")(np.array([n, n], np.int32), grid, out)
    expected = ref.ref_heat2d_gpu(grid)
    # 0.3*c + 0.4*s may be contracted to a fused multiply-add on the GPU
    assert np.max(np.abs(out - expected)) <= 1e-6 * np.max(np.abs(expected))


# ---------------------------------------------------------------- the reference's own GPU tests

@pytest.mark.gpu
@pytest.mark.parametrize("M,N", [(48, 64), (37, 53)])
def test_reference_convolutiongpu(M, N):
    # taps that are multiples of 1/8 and add up to 1: every product and sum is exact and fits uint8
    kernel = np.array([[0, 0.125, 0], [0.125, 0.25, 0.125], [0, 0.25, 0.125]], np.float32)
    img = np.random.RandomState(M + N).randint(0, 256, (3, M, N)).astype(np.uint8)
    out = np.zeros((3, M - 2, N - 2), np.uint8)
    load("convolutiongpu")(np.array([N, M], np.int32), img, kernel, out)
    assert np.array_equal(out, ref.ref_convolution_gpu(img, kernel))


@pytest.mark.gpu
@pytest.mark.parametrize("M,N", [(48, 64), (37, 53), (1, 70), (70, 1)])
def test_reference_fusiongpu(M, N):
    img = np.random.RandomState(M * N).randint(0, 256, (3, M, N)).astype(np.uint8)
    outs = [np.zeros((3, M, N), np.uint8) for _ in range(4)]
    load("fusiongpu")(np.array([N, M], np.int32), img, *outs)
    for got, want in zip(outs, ref.ref_fusion_gpu(img)):
        assert np.array_equal(got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N", [(48, 64), (38, 54)])
def test_reference_rgbyuv420gpu(M, N):
    img = np.random.RandomState(3 * M + N).randint(0, 256, (3, M, N)).astype(np.uint8)
    y, u, v = np.zeros((M, N), np.uint8), np.zeros((M // 2, N // 2), np.uint8), np.zeros((M // 2, N // 2), np.uint8)
    load("rgbyuv420gpu")(np.array([N, M], np.int32), img, y, u, v)
    ey, eu, ev = ref.ref_rgbyuv420_gpu(img)
    assert np.array_equal(y, ey) and np.array_equal(u, eu) and np.array_equal(v, ev)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N", [(96, 128), (75, 101)])
def test_reference_warp_affinegpu(M, N):
    img = np.random.RandomState(M + 7 * N).randint(0, 256, (M, N)).astype(np.uint8)
    out = np.zeros((M, N), np.float32)
    load("warp_affinegpu")(np.array([N, M], np.int32), img, out)
    expected = ref.ref_warp_affine_gpu(img)
    # fused multiply-adds may move a source coordinate that lies on an integer by one ulp to the
    # other side of floor(): such pixels are excused, all others must agree
    f = np.float32
    j, i = np.meshgrid(np.arange(M, dtype=np.float32), np.arange(N, dtype=np.float32), indexing="ij")
    o = (f(0.1) * i + f(0.1) * j).astype(np.float32) + f(0.1)
    on_integer = np.abs(o - np.round(o)) < 1e-4
    ok = np.abs(out - expected) <= 1e-4 * 255
    assert np.all(ok | on_integer)
    assert np.mean(ok) > 0.85


@pytest.mark.gpu
def test_reference_edgegpu():
    # the program is written for 8192 x 8192 x 3 in place (edgegpu_tiramisu.cpp:3-4)
    n = 8192
    img = np.random.RandomState(8192).randint(0, 256, (3, n, n)).astype(np.uint8)
    work = img.copy()
    load("edgegpu")(work)
    assert np.array_equal(work[:, :n - 4, :n - 4], ref.ref_edge_gpu(img))
    assert np.array_equal(work[:, n - 2:, :], img[:, n - 2:, :]) and np.array_equal(work[:, :, n - 2:], img[:, :, n - 2:])


REFERENCE_TESTS = ["wrapper_test_%s" % n for n in ("17", "18", "19", "162", "164", "165", "166", "167", "168", "169", "170", "171", "197")] + \
                  ["wrapper_tutorial_04gpu", "wrapper_tutorial_04gpu2"]


@pytest.mark.parametrize("name", REFERENCE_TESTS)
def test_reference_test_library_exports_its_entry_point(name):
    if not os.path.exists(library(name)):
        pytest.skip("reference tree was absent when the libraries were built")
    runtime.wrappers()
    assert hasattr(ctypes.CDLL(library(name)), "tiramisu_wrapper_main")


@pytest.mark.gpu
@pytest.mark.parametrize("name", REFERENCE_TESTS)
def test_reference_gpu_test_passes(name):
    """Generator (tests/test_N.cpp or the tutorial) and wrapper (wrapper_test_N.cpp) of the reference,
    both unchanged: the wrapper fills Halide::Buffer inputs, calls the generated function, computes
    its own nested-loop expectation and compares (tag_gpu_level / gpu_tile on host buffers without
    gen_cuda_stmt in 17-19: the route of Halide's GPU target in the reference, implicit copies here;
    library GEMM calls in 162-166, gpu_tile and cache_shared GEMMs in 167-171, allocate_at in
    197, uint8 GEMMs in the tutorials).  A mismatch
    ends the process with status 1, as the reference's compare_buffers does."""
    if not os.path.exists(library(name)):
        pytest.skip("reference tree was absent when the libraries were built")
    runtime.wrappers()
    lib = ctypes.CDLL(library(name))
    lib.tiramisu_wrapper_main.restype = ctypes.c_int
    lib.tiramisu_wrapper_main.argtypes = [ctypes.c_int, ctypes.c_void_p]
    print("running", name, flush=True)
    assert lib.tiramisu_wrapper_main(0, None) == 0


DIBARYON = ["gpu_single_tiramisu_make_fused_identical_dibaryon_blocks_correlator", "gpu_tiramisu_make_fused_identical_dibaryon_blocks_correlator"]
BARYON = ["gpu_tiramisu_make_fused_baryon_blocks_correlator", "gpu_tiramisu_make_fused_identical_baryon_blocks_correlator",
          "gpu_single_tiramisu_make_fused_identical_baryon_blocks_correlator"]


@pytest.mark.parametrize("name", BARYON)
def test_reference_baryon_library_exports_its_entry_point(name):
    if not os.path.exists(library(name)):
        pytest.skip("reference tree was absent when the libraries were built")
    runtime.wrappers()
    assert hasattr(ctypes.CDLL(library(name)), "tiramisu_wrapper_main")


@pytest.mark.gpu
@pytest.mark.parametrize("name", BARYON)
def test_reference_baryon_correlator_passes_its_own_check(name):
    """benchmarks/tensors/baryon/gpu_*: generator and wrapper of the reference, both unchanged.  The wrapper fills
    random propagators, wave functions and weights, runs the generated function (six kernels in complex fp64) and
    the C++ restatement that the reference keeps next to it, and compares every correlator entry to a relative
    1e-12; on a difference it ends the process with status 1."""
    if not os.path.exists(library(name)):
        pytest.skip("reference tree was absent when the libraries were built")
    runtime.wrappers()
    lib = ctypes.CDLL(library(name))
    lib.tiramisu_wrapper_main.restype = ctypes.c_int
    lib.tiramisu_wrapper_main.argtypes = [ctypes.c_int, ctypes.c_void_p]
    print("running", name, flush=True)
    assert lib.tiramisu_wrapper_main(0, None) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("name", DIBARYON)
def test_reference_dibaryon_correlator_passes_its_own_check(name):
    """benchmarks/tensors/dibaryon/gpu_single_...: generator unchanged; the wrapper with its two switches
    (RUN_REFERENCE, RUN_CHECK) on, so that it runs the authors' C++ restatement and compares every correlator entry
    with the generated function's (ten kernels; kernels inside host loops take the loops' iterators as parameters
    in a program with 64-bit loop iterators; in the second program statements tagged (block, thread) are fused at
    their second level with statements tagged (block, block, thread, thread), and their accumulations have no
    thread loop around them).  Built on request only (TIRAMISU_BUILD_DIBARYON=1: about ten minutes each)."""
    if not os.path.exists(library(name)):
        pytest.skip("built on request only: TIRAMISU_BUILD_DIBARYON=1 python tests/reference_programs/build_reference_programs.py")
    if os.environ.get("TIRAMISU_RUN_DIBARYON") != "1":
        pytest.skip("a minute and a half each, most of it the wrapper's own set-up on the host: run with TIRAMISU_RUN_DIBARYON=1")
    runtime.wrappers()
    lib = ctypes.CDLL(library(name))
    lib.tiramisu_wrapper_main.restype = ctypes.c_int
    lib.tiramisu_wrapper_main.argtypes = [ctypes.c_int, ctypes.c_void_p]
    print("running", name, flush=True)
    here = os.getcwd()
    work = os.path.join(HERE, "reference_programs", "build", name)
    os.chdir(work)                      # the wrapper writes performance_CPU.csv where it runs
    try:
        assert lib.tiramisu_wrapper_main(0, None) == 0
    finally:
        os.chdir(here)


TUNED_SGEMM = {"sgemm_generator1": "generic", "sgemm_generator2": "generic", "sgemm_generator3": "mfma-contraction"}


@pytest.mark.parametrize("name", sorted(TUNED_SGEMM))
def test_reference_tuned_sgemm_library(name):
    """The hand-staged schedules stay as scheduled; the cache_shared one is proven a dense
    contraction (LDS tiles cover their reads, register tile private) and gets the MFMA kernel."""
    if not os.path.exists(library(name)):
        pytest.skip("reference tree was absent when the libraries were built")
    runtime.wrappers()
    ctypes.CDLL(library("get_time"), mode=ctypes.RTLD_GLOBAL)
    assert hasattr(ctypes.CDLL(library(name)), "matmul")
    text = open(os.path.join(HERE, "reference_programs", "build", name, "fct.o.hip")).read()
    assert ("// _kernel_0: " + TUNED_SGEMM[name]) in text


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(TUNED_SGEMM))
def test_reference_tuned_sgemm_schedule(name):
    """benchmarks/linear_algebra/blas/level3/sgemm/gpu/generator{1,2,3}.cpp, unchanged: 3072^3 with a
    16x6 (16x8 in generator3) register tile per thread and LDS tiles of both operands, staged by
    hand in generator1 (double-buffered) and generator2, with cache_shared in generator3.  Each
    copies A, B, C to the GPU, times its kernel with get_time() and copies C back.  Their wrapper
    needs CUDA headers, so the generated function is called here; small integer data keeps every
    sum exact, so the comparison with a float64 product is for equality."""
    if not os.path.exists(library(name)):
        pytest.skip("reference tree was absent when the libraries were built")
    ctypes.CDLL(library("get_time"), mode=ctypes.RTLD_GLOBAL)
    program = runtime.Program(library(name), "matmul")
    n = 3072
    rng = np.random.RandomState(3072)
    A = rng.randint(-2, 3, (n, n)).astype(np.float32)
    B = rng.randint(-2, 3, (n, n)).astype(np.float32)
    C0 = rng.randint(-4, 5, (n, n)).astype(np.float32)
    consts = np.array([3, 2], np.float32)
    expected = (3.0 * (A.astype(np.float64) @ B.astype(np.float64)) + 2.0 * C0).astype(np.float32)
    import time
    best = whole = None
    for _ in range(3):
        C = C0.copy()
        t0, t1 = np.zeros(1, np.float32), np.zeros(1, np.float32)
        start = time.perf_counter()
        program(consts, A, B, C, t0, t1)
        call_ms = (time.perf_counter() - start) * 1e3
        assert np.array_equal(C, expected)
        ms = float(t1[0] - t0[0])
        best = ms if best is None else min(best, ms)
        whole = call_ms if whole is None else min(whole, call_ms)
    print("%s kernel: %.3f ms, %.1f TFLOP/s; whole call with allocation and copies: %.2f ms"
          % (name, best, 2.0 * n ** 3 / best / 1e9, whole), flush=True)


def lstm_inputs(L, B, H, S, seed):
    rng = np.random.RandomState(seed)
    bound = 1.0 / np.sqrt(H)
    weights = rng.uniform(-bound, bound, (L, 2, 4 * H, H)).astype(np.float32)
    biases = rng.uniform(-bound, bound, (L, 4 * H)).astype(np.float32)
    x = rng.uniform(-1, 1, (S, B, H)).astype(np.float32)
    return weights, biases, x


@pytest.mark.parametrize("name", ["lstm_gpu", "lstm_gpu_lib", "lstm_gpu_lib_f64"])
def test_reference_lstm_library_exports_its_function(name):
    """Both GPU LSTM generators compile and generate code unchanged.  Only gpu_lib's function is
    run: gpu/generator.cpp maps its reads of the previous hidden state to rows {m - 1, l} of the
    state buffer (:268, :280) while the states are stored at {m + 1, l + 1} (:295), so its first
    step reads row -1, before the allocation."""
    if not os.path.exists(library(name)):
        pytest.skip("reference tree was absent when the libraries were built")
    runtime.wrappers()
    ctypes.CDLL(library("get_time"), mode=ctypes.RTLD_GLOBAL)
    assert hasattr(ctypes.CDLL(library(name)), "lstm")


@pytest.mark.gpu
def test_reference_lstm_gpu_lib_generator():
    """benchmarks/DNN/blocks/LSTM/gpu_lib/generator.cpp, unchanged, at its own size (4 layers, batch
    64, 512 features, 100 steps): weights transposed on the GPU, library GEMM calls with offsets
    (input products batched over 10 steps), (layer, step block) walked diagonally after skew +
    interchange, nonlinearities in one fused kernel per step.  The program times itself."""
    if not os.path.exists(library("lstm_gpu_lib")):
        pytest.skip("reference tree was absent when the libraries were built")
    ctypes.CDLL(library("get_time"), mode=ctypes.RTLD_GLOBAL)
    L, B, H, S = 4, 64, 512, 100
    weights, biases, x = lstm_inputs(L, B, H, S, 512)
    program = runtime.Program(library("lstm_gpu_lib"), "lstm")
    expected = ref.lstm(weights, biases, x)
    import time
    best = whole = None
    for _ in range(3):
        y = np.zeros((S, B, H), np.float32)
        t0, t1 = np.zeros(1, np.float32), np.zeros(1, np.float32)
        start = time.perf_counter()
        program(weights, biases, x, y, t0, t1)
        call_ms = (time.perf_counter() - start) * 1e3
        assert np.max(np.abs(y - expected)) <= 1e-4 * np.max(np.abs(expected))
        ms = float(t1[0] - t0[0])
        best = ms if best is None else min(best, ms)
        whole = call_ms if whole is None else min(whole, call_ms)
    print("gpu_lib LSTM generator: %.3f ms between its timers, %.3f ms for the whole call with allocation and copies"
          % (best, whole), flush=True)


@pytest.mark.gpu
def test_reference_lstm_gpu_lib_generator_in_double_precision():
    """The same generator with its configuration switched to double precision (the switch of the reference's
    gpu_lib/configuration.h, flipped while the program is compiled): the products go through
    tiramisu_hip_dgemm (fp64 matrix instructions), the rest through the generic emitter on doubles.  The
    reference publishes 106.7 ms for this on a K80 (gpu_lib/README.md:7-14)."""
    if not os.path.exists(library("lstm_gpu_lib_f64")):
        pytest.skip("reference tree was absent when the libraries were built")
    ctypes.CDLL(library("get_time"), mode=ctypes.RTLD_GLOBAL)
    L, B, H, S = 4, 64, 512, 100
    weights, biases, x = (a.astype(np.float64) for a in lstm_inputs(L, B, H, S, 512))
    program = runtime.Program(library("lstm_gpu_lib_f64"), "lstm")
    expected = ref.lstm(weights, biases, x, real=np.float64)
    import time
    best = whole = None
    for _ in range(3):
        y = np.zeros((S, B, H), np.float64)
        t0, t1 = np.zeros(1, np.float32), np.zeros(1, np.float32)
        start = time.perf_counter()
        program(weights, biases, x, y, t0, t1)
        call_ms = (time.perf_counter() - start) * 1e3
        assert np.max(np.abs(y - expected)) <= 1e-9 * np.max(np.abs(expected))
        ms = float(t1[0] - t0[0])
        best = ms if best is None else min(best, ms)
        whole = call_ms if whole is None else min(whole, call_ms)
    print("gpu_lib LSTM generator in double precision: %.3f ms between its timers, %.3f ms for the whole call with allocation and copies"
          % (best, whole), flush=True)


def test_reference_chain_mm_library_exports_its_function():
    if not os.path.exists(library("chain_mm")):
        pytest.skip("reference tree was absent when the libraries were built")
    runtime.wrappers()
    assert hasattr(ctypes.CDLL(library("chain_mm")), "matmul")
    text = open(os.path.join(HERE, "reference_programs", "build", "chain_mm", "fct.o.hip")).read()
    assert text.count("mfma-contraction") == 2


@pytest.mark.gpu
def test_reference_chain_mm_generator():
    """benchmarks/linear_algebra/chain_mm/gpu/generator.cpp, unchanged: O = (A x B) x C with
    1024x512, 512x128 and 128x256 operands (configuration.h), each product a gpu_tile nest with its
    zero initialisation fused at the thread level; both become MFMA kernels.  Integer data small
    enough that every partial sum is exact in fp32."""
    if not os.path.exists(library("chain_mm")):
        pytest.skip("reference tree was absent when the libraries were built")
    rng = np.random.RandomState(1024)
    A = rng.randint(-2, 3, (1024, 512)).astype(np.float32)
    B = rng.randint(-2, 3, (512, 128)).astype(np.float32)
    C = rng.randint(-2, 3, (128, 256)).astype(np.float32)
    O = np.full((1024, 256), -1, np.float32)
    runtime.Program(library("chain_mm"), "matmul")(A, B, C, O)
    expected = ((A.astype(np.float64) @ B.astype(np.float64)) @ C.astype(np.float64)).astype(np.float32)
    assert np.array_equal(O, expected)


@pytest.mark.parametrize("L,B,H,S", [(2, 3, 8, 4), (1, 2, 5, 3), (3, 4, 6, 2)])
def test_naive_lstm_program_pins_the_packing(L, B, H, S):
    """benchmarks/DNN/blocks/LSTM/gpu/reference_generator.cpp, unchanged (a CPU program: four separate gate sums with
    explicit loops, sizes at run time), compiled through the oracle's CPU emitter: its output must be
    what the numpy oracle computes once the buffers are re-packed from the GPU generators' layout
    (slot 0 = R, rows i, z, o, f).  Summation order differs (a j loop here, matrix products there)."""
    if not os.path.exists(library("lstm_ref")):
        pytest.skip("reference tree was absent when the libraries were built")
    rng = np.random.RandomState(10 * L + H)
    weights = rng.uniform(-0.5, 0.5, (L, 2, 4 * H, H)).astype(np.float32)
    biases = rng.uniform(-0.5, 0.5, (L, 4 * H)).astype(np.float32)
    x = rng.uniform(-1, 1, (S, B, H)).astype(np.float32)
    y = np.zeros((S, B, H), np.float32)
    runtime.Program(library("lstm_ref"), "lstm_ref", needs_gpu_runtime=False)(np.array([H, B, L, S], np.int32), weights, biases, x, y)
    expected = ref.lstm_gpu_packing(weights, biases, x)
    assert np.max(np.abs(y - expected)) <= 2e-6
    # and the packing matters: without the re-packing the result is a different one
    assert np.max(np.abs(y - ref.lstm(weights, biases, x))) > 1e-3
