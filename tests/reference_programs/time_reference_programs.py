"""Times the GPU benchmark programs of the reference tree that this build compiles unchanged
(build_reference_programs.py) on the GPU of this machine, at the sizes their own wrappers use:
the eight image pipelines of benchmarks/halide on a 2112 x 3520 image (the size of the tree's
utils/images; heat2dgpu on its wrapper's 10000 x 10000 grid, edgegpu on the 8192 x 8192 x 3 it is
written for), the three tuned sgemm schedules, chain_mm, the library LSTM (configuration 5's shape) and the three baryon
correlators (through their own wrappers).  The programs copy to and from the GPU
themselves; what is timed is their kernels: HIP events around every launch of a call
(tiramisu_hip_profile_*), median over the calls.  Bytes are the algorithmic ones: every input and
output element once.  Prints one markdown table.  Run from the repository root on a machine with a
GPU, for all programs or for those named:
    python tests/reference_programs/time_reference_programs.py [program ...]
"""
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from tiramisu_amd import runtime  # noqa: E402

HBM_PEAK_GBS, FP32_MFMA_PEAK_TFLOPS = 8000.0, 157.3
CALLS = 7


BUILD = os.environ.get("TIRAMISU_REFERENCE_PROGRAMS_BUILD", os.path.join(HERE, "build"))   # where the libraries lie


def library(name):
    return os.path.join(BUILD, "lib%s.so" % name)


def kernel_times(call):
    """[(sum of the kernels of one call in ms, {kernel: (ms, launches)})], median call by the sum."""
    runs = []
    for _ in range(CALLS):
        by = {}
        for name, ms in runtime.profile(call):
            t, n = by.get(name, (0.0, 0))
            by[name] = (t + ms, n + 1)
        runs.append((sum(t for t, _ in by.values()), by))
    runs.sort(key=lambda r: r[0])
    return runs[len(runs) // 2]


def image_pipelines(only):
    M, N = 3520, 2112                       # rows, columns
    rng = np.random.RandomState(1)
    rgb = rng.randint(0, 256, (3, M, N)).astype(np.uint8)
    gray = rgb[0].copy()
    out = []

    def add(name, function, args, nbytes, note):
        if only and name not in only:
            return
        program = runtime.Program(library(name), function)
        program(*args)                      # first call: module load
        total, by = kernel_times(lambda: program(*args))
        out.append((name, note, total, by, nbytes))

    add("cvtcolorgpu", "cvtcolorgpu_tiramisu", (np.array([N, M], np.int32), rgb, np.zeros((M, N), np.uint8)), 4 * M * N,
        "RGB to gray, uint8, %dx%d" % (N, M))
    kx = np.array([1, 4, 6, 4, 1], np.float32)
    add("gaussiangpu", "gaussiangpu_tiramisu", (np.array([N, M, 3], np.int32), rgb, kx, kx / np.float32(256), np.zeros((3, M - 5, N - 5), np.uint8)),
        3 * M * N + 3 * (M - 5) * (N - 5), "separable 5-tap blur, uint8, 3 channels (two passes: the intermediate is read and written as well)")
    kernel = np.array([[0, 0.125, 0], [0.125, 0.25, 0.125], [0, 0.25, 0.125]], np.float32)
    add("convolutiongpu", "convolutiongpu_tiramisu", (np.array([N, M], np.int32), rgb, kernel, np.zeros((3, M - 2, N - 2), np.uint8)),
        3 * M * N + 3 * (M - 2) * (N - 2), "3x3 filter, uint8, 3 channels")
    add("fusiongpu", "fusiongpu_tiramisu", (np.array([N, M], np.int32), rgb) + tuple(np.zeros((3, M, N), np.uint8) for _ in range(4)),
        5 * 3 * M * N, "four point-wise outputs of one input, uint8")
    add("rgbyuv420gpu", "rgbyuv420gpu_tiramisu",
        (np.array([N, M], np.int32), rgb, np.zeros((M, N), np.uint8), np.zeros((M // 2, N // 2), np.uint8), np.zeros((M // 2, N // 2), np.uint8)),
        3 * M * N + M * N + 2 * (M // 2) * (N // 2), "RGB to YUV 4:2:0, uint8")
    add("warp_affinegpu", "warp_affinegpu_tiramisu", (np.array([N, M], np.int32), gray, np.zeros((M, N), np.float32)), M * N + 4 * M * N,
        "affine warp with bilinear interpolation, uint8 to float")
    n = 10000
    grid = rng.uniform(0, 1, (n, n)).astype(np.float32)
    add("heat2dgpu", "heat2dgpu_tiramisu", (np.array([n, n], np.int32), grid, np.zeros((n, n), np.float32)), 2 * 4 * n * n,
        "one 5-point sweep, float, %dx%d, 32x32 LDS tiles staged by the program" % (n, n))
    n = 8192
    img = rng.randint(0, 256, (3, n, n)).astype(np.uint8)
    add("edgegpu", "edge_tiramisu", (img,), 2 * 2 * 3 * n * n, "two 3x3 passes in place, uint8, %dx%dx3" % (n, n))
    return out


def gemm_programs(only):
    out = []
    if only and not any(o.startswith("sgemm") or o == "chain_mm" for o in only):
        return out
    ctypes.CDLL(library("get_time"), mode=ctypes.RTLD_GLOBAL)
    n = 3072
    rng = np.random.RandomState(3072)
    A, B, C = (rng.uniform(-1, 1, (n, n)).astype(np.float32) for _ in range(3))
    consts = np.array([3, 2], np.float32)
    for g in (1, 2, 3):
        if only and "sgemm_generator%d" % g not in only:
            continue
        program = runtime.Program(library("sgemm_generator%d" % g), "matmul")
        t0, t1 = np.zeros(1, np.float32), np.zeros(1, np.float32)
        args = (consts, A, B, C.copy(), t0, t1)
        program(*args)
        total, by = kernel_times(lambda: program(*args))
        out.append(("sgemm generator%d" % g, "3072^3, %s" % ("explicit LDS copies, double-buffered" if g == 1 else "explicit LDS copies" if g == 2 else "cache_shared"),
                    total, by, 2.0 * n ** 3))
    if not only or "chain_mm" in only:
        rng = np.random.RandomState(1024)
        A2, B2, C2 = (rng.uniform(-1, 1, shape).astype(np.float32) for shape in ((1024, 512), (512, 128), (128, 256)))
        O = np.zeros((1024, 256), np.float32)
        program = runtime.Program(library("chain_mm"), "matmul")
        program(A2, B2, C2, O)
        total, by = kernel_times(lambda: program(A2, B2, C2, O))
        out.append(("chain_mm", "(1024x512 x 512x128) x 128x256, two gpu_tile nests", total, by, 2.0 * 1024 * 128 * (512 + 256)))
    return out


BARYON = ["gpu_tiramisu_make_fused_baryon_blocks_correlator", "gpu_tiramisu_make_fused_identical_baryon_blocks_correlator",
          "gpu_single_tiramisu_make_fused_identical_baryon_blocks_correlator"]


def correlator_programs(only):
    """The baryon correlator benchmarks, run by their own wrappers (which also run the reference's C++ restatement
    and compare): the kernels of the generated function, at the lattice size the reference's parameter header sets."""
    out = []
    for name in BARYON:
        if only and name not in only:
            continue
        lib = ctypes.CDLL(library(name))
        lib.tiramisu_wrapper_main.restype = ctypes.c_int
        lib.tiramisu_wrapper_main.argtypes = [ctypes.c_int, ctypes.c_void_p]

        def call():
            # the wrapper prints every correlator entry: keep that out of the table
            sys.stdout.flush()
            saved, null = os.dup(1), os.open(os.devnull, os.O_WRONLY)
            os.dup2(null, 1)
            try:
                status = lib.tiramisu_wrapper_main(0, None)
            finally:
                os.dup2(saved, 1)
                os.close(saved)
                os.close(null)
            assert status == 0
        call()
        total, by = kernel_times(call)
        out.append((name, total, by))
    return out


def lstm_program(only):
    """benchmarks/DNN/blocks/LSTM/gpu_lib/generator.cpp, unchanged: 4 layers, batch 64, 512 features, 100 steps.  The
    program times itself between its device copies (get_time(), timer_hook.c); the kernels of the same call by HIP
    events (events between the launches of a dependent chain cost a good part of a launch themselves, so their sum
    is above the program's own figure)."""
    name = "lstm_gpu_lib"
    if (only and name not in only) or not os.path.exists(library(name)):
        return []
    ctypes.CDLL(library("get_time"), mode=ctypes.RTLD_GLOBAL)
    L, B, H, S = 4, 64, 512, 100
    rng = np.random.RandomState(5)
    weights = rng.uniform(-0.08, 0.08, (L, 2, 4 * H, H)).astype(np.float32)
    biases = rng.uniform(-0.08, 0.08, (L, 4 * H)).astype(np.float32)
    x = rng.uniform(-1, 1, (S, B, H)).astype(np.float32)
    program = runtime.Program(library(name), "lstm")
    y, t0, t1 = np.zeros((S, B, H), np.float32), np.zeros(1, np.float32), np.zeros(1, np.float32)
    own = []
    for _ in range(CALLS + 1):
        program(weights, biases, x, y, t0, t1)
        own.append(float(t1[0] - t0[0]))
    total, by = kernel_times(lambda: program(weights, biases, x, y, t0, t1))
    return [(name, "4-layer LSTM, batch 64, 512 features, 100 steps: library GEMMs + one point-wise kernel per step", sorted(own[1:])[CALLS // 2], total, by,
             L * S * 2 * (2.0 * B * 4 * H * H))]


def main():
    only = set(sys.argv[1:])
    runtime.wrappers()
    print("| program | what | kernels of one call | time | algorithmic rate | of the roofline |")
    print("|---|---|---|---|---|---|")
    for name, note, total, by, nbytes in image_pipelines(only):
        kernels = ", ".join("%s %.1f us%s" % (k, t / n * 1e3, " x %d" % n if n > 1 else "") for k, (t, n) in sorted(by.items()))
        gbs = nbytes / (total * 1e-3) / 1e9
        print("| `%s` | %s | %s | %.3f ms | %.0f GB/s | %.2f of 8 TB/s |" % (name, note, kernels, total, gbs, gbs / HBM_PEAK_GBS), flush=True)
    for name, total, by in correlator_programs(only):
        kernels = ", ".join("%s %.1f us%s" % (k, t / n * 1e3, " x %d" % n if n > 1 else "") for k, (t, n) in sorted(by.items()))
        print("| `%s` | complex fp64 contractions, the reference's parameter set; checked by the wrapper against the reference's C++ | %s | %.3f ms | - | - |"
              % (name, kernels, total), flush=True)
    for name, note, total, by, flop in gemm_programs(only):
        kernels = ", ".join("%s %.3f ms" % (k, t / n) for k, (t, n) in sorted(by.items()))
        tf = flop / (total * 1e-3) / 1e12
        print("| %s | %s | %s | %.3f ms | %.1f TFLOP/s | %.2f of %.1f TFLOP/s |" % (name, note, kernels, total, tf, tf / FP32_MFMA_PEAK_TFLOPS, FP32_MFMA_PEAK_TFLOPS), flush=True)
    for name, note, own_ms, total, by, flop in lstm_program(only):
        kernels = ", ".join("%s %.1f us x %d" % (k, t / n * 1e3, n) for k, (t, n) in sorted(by.items()))
        tf = flop / (own_ms * 1e-3) / 1e12
        print("| `%s` | %s | %s (sum between events %.3f ms) | %.3f ms between the program's own timers | %.1f TFLOP/s | %.2f of %.1f TFLOP/s |"
              % (name, note, kernels, total, own_ms, tf, tf / FP32_MFMA_PEAK_TFLOPS, FP32_MFMA_PEAK_TFLOPS), flush=True)


if __name__ == "__main__":
    main()
