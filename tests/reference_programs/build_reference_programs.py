"""Compiles GPU generator programs of the reference tree, *unchanged*, against this build's headers
and compiler library, and links the functions they generate -- the strongest form of the drop-in
claim: the reference's own Tiramisu programs (isl-string domains, low-level pipeline, constants,
shared and constant memory, inlining) go through the HIP back-end as they are.

The sources are read where they lie (/root/reference, never copied); everything written goes to
tests/reference_programs/build/.  Where the reference tree is absent (the GPU box) nothing is built
and the tests use the libraries built beforehand.  Run from the repository root:
    python tests/reference_programs/build_reference_programs.py
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from tiramisu_amd import build  # noqa: E402

REFERENCE = os.environ.get("TIRAMISU_REFERENCE_TREE", "/root/reference")

# (source below the reference tree, preprocessor defines its CMake build passes, generated function)
PROGRAMS = [
    ("benchmarks/halide/cvtcolorgpu_tiramisu.cpp", [], "cvtcolorgpu"),
    ("benchmarks/halide/gaussiangpu_tiramisu.cpp", [], "gaussiangpu"),
    ("benchmarks/halide/heat2dgpu_tiramisu.cpp", ["USE_GPU2"], "heat2dgpu"),
    ("benchmarks/halide/convolutiongpu_tiramisu.cpp", [], "convolutiongpu"),
    ("benchmarks/halide/fusiongpu_tiramisu.cpp", [], "fusiongpu"),
    ("benchmarks/halide/rgbyuv420gpu_tiramisu.cpp", [], "rgbyuv420gpu"),
    ("benchmarks/halide/warp_affinegpu_tiramisu.cpp", [], "warp_affinegpu"),
    ("benchmarks/halide/edgegpu_tiramisu.cpp", [], "edgegpu"),
]


# The reference's own GPU tests and tutorials: generator and wrapper program, both unchanged.
# The wrapper (main(): Halide::Buffer inputs, nested-loop expectation, compare_buffers) is linked
# with the object its generator wrote into build/lib<wrapper>.so and run in-process by the tests.
# (generator, wrapper) below the reference tree:
TESTS = [("tests/test_%s.cpp" % n, "tests/wrapper_test_%s.cpp" % n)
         for n in ("17", "18", "19", "162", "164", "165", "166", "167", "168", "169", "170", "171", "197")] + [
    ("tutorials/developers/tutorial_04gpu/tutorial_04gpu.cpp", "tutorials/developers/tutorial_04gpu/wrapper_tutorial_04gpu.cpp"),
    ("tutorials/developers/tutorial_04gpu2/tutorial_04gpu2.cpp", "tutorials/developers/tutorial_04gpu2/wrapper_tutorial_04gpu2.cpp"),
]


def library(name):
    return os.path.join(HERE, "build", "lib%s.so" % name)


def wrapper_name(wrapper_rel):
    return os.path.splitext(os.path.basename(wrapper_rel))[0]


def build_test(generator_rel, wrapper_rel):
    bdir = os.path.join(HERE, "build")
    produced = build.build_program(os.path.join(REFERENCE, generator_rel), directory=HERE, shim_headers=True) or []
    objects = [os.path.join(bdir, o) for o in produced]
    entry = os.path.join(bdir, "entry.h")
    with open(entry, "w") as f:
        f.write('extern "C" int tiramisu_wrapper_main(int, char **);\n')
    wrapper = os.path.join(REFERENCE, wrapper_rel)
    build._run(["g++", "-std=c++17", "-O1", "-fPIC", "-shared", "-I" + build.INCLUDE,
                "-I" + os.path.join(build.INCLUDE, "tiramisu", "shim"), "-I" + os.path.dirname(wrapper),
                "-include", entry, "-Dmain=tiramisu_wrapper_main", "-o", library(wrapper_name(wrapper_rel)), wrapper] + objects +
               ["-L" + build.PKG, "-ltiramisu_hip_wrappers", "-Wl,-rpath,$ORIGIN/" + os.path.relpath(build.PKG, bdir)])


# Benchmark generators whose wrapper needs CUDA, cuBLAS or cuDNN headers: the tests drive the
# generated function themselves.  Each program writes its object into its working directory and
# (all but the first LSTM) times its kernels through an external get_time(): timer_hook.c.
#  * sgemm at 3072^3: generator1 and generator2 stage the operands by hand (explicit LDS copies,
#    double-buffered in generator1; 16x6 register tile), generator3 uses cache_shared (16x8).
#  * LSTM: gpu/generator.cpp takes its sizes at run time and stages both matrix products through
#    LDS by hand; gpu_lib/generator.cpp (4 layers, batch 64, 512 features, 100 steps) calls the
#    library GEMM, batches the input products over 10 steps and walks (layer, step block)
#    diagonally with skew + interchange under a parallel host loop.
#  * chain_mm: (A x B) x C, two GEMM nests with the reduction loop interchanged inward.
# (source below the reference tree, library stem, object the program writes):
SELF_DRIVEN = [("benchmarks/linear_algebra/blas/level3/sgemm/gpu/generator%d.cpp" % n, "sgemm_generator%d" % n, "fct.o")
               for n in (1, 2, 3)] + [
    ("benchmarks/DNN/blocks/LSTM/gpu/generator.cpp", "lstm_gpu", "lstm.o"),
    ("benchmarks/DNN/blocks/LSTM/gpu_lib/generator.cpp", "lstm_gpu_lib", "lstm.o"),
    ("benchmarks/linear_algebra/chain_mm/gpu/generator.cpp", "chain_mm", "fct.o"),
]


def build_self_driven(rel, stem, obj):
    bdir = os.path.join(HERE, "build")
    work = os.path.join(bdir, stem)
    os.makedirs(work, exist_ok=True)
    src = os.path.join(REFERENCE, rel)
    gen = os.path.join(work, "gen")
    build._run(["g++", "-std=c++17", "-O1", "-I" + build.INCLUDE, "-I" + os.path.join(build.INCLUDE, "tiramisu", "shim"),
                "-I" + os.path.dirname(src), "-o", gen, src, "-L" + build.PKG, "-ltiramisu", "-Wl,-rpath," + build.PKG])
    build._run([gen], cwd=work)
    build._run(["gcc", "-O2", "-fPIC", "-shared", "-o", library("get_time"), os.path.join(HERE, "timer_hook.c")])
    build._run(["g++", "-shared", "-o", library(stem), os.path.join(work, obj), "-L" + build.PKG,
                "-ltiramisu_hip_wrappers", "-Wl,-rpath,$ORIGIN/" + os.path.relpath(build.PKG, bdir)])


# The reference's naive restatement of its LSTM (a CPU program: codegen without the GPU flag), compiled
# unchanged through the oracle's CPU emitter: the pin of the numpy LSTM oracle's packing and gate order
# for the reference's GPU generator (slot 0 = R, rows i, z, o, f).
LSTM_NAIVE = "benchmarks/DNN/blocks/LSTM/gpu/reference_generator.cpp"


def build_lstm_naive():
    from oracle import build as oracle_build
    bdir = os.path.join(HERE, "build")
    work = os.path.join(bdir, "lstm_ref")
    os.makedirs(work, exist_ok=True)
    src = os.path.join(REFERENCE, LSTM_NAIVE)
    gen = os.path.join(work, "gen")
    cpu_dir = os.path.dirname(oracle_build.CPU_BACKEND)
    build._run(["g++", "-std=c++17", "-O1", "-I" + build.INCLUDE, "-I" + os.path.join(build.INCLUDE, "tiramisu", "shim"), "-o", gen, src,
                "-L" + build.PKG, "-ltiramisu", "-Wl,--no-as-needed", "-L" + cpu_dir, "-ltiramisu_cpu_backend", "-Wl,--as-needed",
                "-Wl,-rpath," + build.PKG, "-Wl,-rpath," + cpu_dir])
    build._run([gen], cwd=work)
    build._run(["g++", "-shared", "-fopenmp", "-o", library("lstm_ref"), os.path.join(work, "lstm_ref.o")])


def build_all(verbose=False):
    if not os.path.isdir(REFERENCE):
        if verbose:
            print("[reference programs] %s is absent: nothing built" % REFERENCE)
        return False
    for rel, defines, name in PROGRAMS:
        if verbose:
            print("[reference programs]", rel, flush=True)
        build.build_program(os.path.join(REFERENCE, rel), defines=defines, directory=HERE, shim_headers=True)
    for generator_rel, wrapper_rel in TESTS:
        if verbose:
            print("[reference programs]", generator_rel, "+", os.path.basename(wrapper_rel), flush=True)
        build_test(generator_rel, wrapper_rel)
    for rel, stem, obj in SELF_DRIVEN:
        if verbose:
            print("[reference programs]", rel, flush=True)
        build_self_driven(rel, stem, obj)
    if verbose:
        print("[reference programs]", LSTM_NAIVE, "(CPU)", flush=True)
    build_lstm_naive()
    return True


if __name__ == "__main__":
    build_all(verbose=True)
