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


# The lattice-QCD correlator benchmarks for the GPU whose code this build generates in seconds (complex fp64
# arithmetic through utils/complex_util.h, six kernels each; the dibaryon programs are further down).  Each wrapper fills random propagators and wave functions, calls the
# generated function and the plain C++ restatement its authors wrote next to it (<...>_ref.cpp, which the wrapper
# includes), and compares the correlators to a relative 1e-12.  Built like the tests above: generator unchanged,
# wrapper unchanged, its main() renamed so that a test can call it in-process.
BARYON = ["benchmarks/tensors/baryon/gpu_tiramisu_make_fused_baryon_blocks_correlator",
          "benchmarks/tensors/baryon/gpu_tiramisu_make_fused_identical_baryon_blocks_correlator",
          "benchmarks/tensors/baryon/gpu_single_tiramisu_make_fused_identical_baryon_blocks_correlator"]


def build_baryon(rel):
    name = os.path.basename(rel)
    source = os.path.join(REFERENCE, rel)
    bdir = os.path.join(HERE, "build")
    work = os.path.join(bdir, name)                  # the generator writes generated_<name>.o where it runs
    os.makedirs(work, exist_ok=True)
    generator = [f for f in os.listdir(source) if f.endswith("_generator.cpp")][0]
    wrapper = [f for f in os.listdir(source) if f.endswith("_wrapper.cpp")][0]
    build.build_program(os.path.join(source, generator), directory=work, shim_headers=True)
    objects = [os.path.join(work, f) for f in os.listdir(work) if f.endswith(".o")]
    entry = os.path.join(bdir, "entry.h")
    with open(entry, "w") as f:
        f.write('extern "C" int tiramisu_wrapper_main(int, char **);\n')
    build._run(["g++", "-std=c++17", "-O2", "-w", "-fPIC", "-shared", "-I" + build.INCLUDE,
                "-I" + os.path.join(build.INCLUDE, "tiramisu", "shim"), "-I" + source,
                "-include", entry, "-Dmain=tiramisu_wrapper_main", "-o", library(name), os.path.join(source, wrapper)] + objects +
               ["-L" + build.PKG, "-ltiramisu_hip_wrappers", "-Wl,-rpath,$ORIGIN/" + os.path.relpath(build.PKG, bdir)])


# Two of the four dibaryon correlators (benchmarks/tensors/dibaryon/gpu_*): ten kernels, 1.3 MB of kernel source each.  (The other
# two build the same way -- build_dibaryon takes any of them -- but the one tried did not finish within ten minutes on the GPU.)
# Compiling a generator takes four minutes and running it one (almost five with the AST built from the flat
# schedule map: three quarters of that inside isl's ordering of the statements' domains), so it is built on request
# only: TIRAMISU_BUILD_DIBARYON=1.
# Each wrapper keeps the comparison with the authors' C++ restatement behind two switches that are off
# ("#define RUN_REFERENCE 0", "#define RUN_CHECK 0") and includes that restatement, standard headers and all, inside
# an extern "C" block: the switches are flipped on the way into the compiler (the text goes through a pipe; nothing of
# the reference is written anywhere) and the standard headers are included ahead of the file.
DIBARYON = ["benchmarks/tensors/dibaryon/gpu_single_tiramisu_make_fused_identical_dibaryon_blocks_correlator",
            "benchmarks/tensors/dibaryon/gpu_tiramisu_make_fused_identical_dibaryon_blocks_correlator"]


def build_dibaryon(rel):
    import subprocess
    name = os.path.basename(rel)
    source = os.path.join(REFERENCE, rel)
    bdir = os.path.join(HERE, "build")
    work = os.path.join(bdir, name)
    os.makedirs(work, exist_ok=True)
    generator = [f for f in os.listdir(source) if f.endswith("_generator.cpp")][0]
    wrapper = [f for f in os.listdir(source) if f.endswith("_wrapper.cpp")][0]
    # the AST from the schedule as a tree: 55 s of generation instead of 4 min 40 s (back-end option ast_from_schedule_tree)
    before = os.environ.get("TIRAMISU_AST_FROM_SCHEDULE_TREE")
    os.environ["TIRAMISU_AST_FROM_SCHEDULE_TREE"] = "1"
    try:
        build.build_program(os.path.join(source, generator), directory=work, shim_headers=True)
    finally:
        if before is None:
            del os.environ["TIRAMISU_AST_FROM_SCHEDULE_TREE"]
        else:
            os.environ["TIRAMISU_AST_FROM_SCHEDULE_TREE"] = before
    objects = [os.path.join(work, f) for f in os.listdir(work) if f.endswith(".o")]
    entry = os.path.join(bdir, "entry.h")
    with open(entry, "w") as f:
        f.write('extern "C" int tiramisu_wrapper_main(int, char **);\n')
    text = open(os.path.join(source, wrapper)).read()
    for switch in ("RUN_REFERENCE", "RUN_CHECK"):
        if "#define %s 0" % switch not in text:
            raise RuntimeError("%s: no '#define %s 0' to flip" % (wrapper, switch))
        text = text.replace("#define %s 0" % switch, "#define %s 1" % switch)
    ahead = []
    for h in ("complex", "vector", "fstream", "string", "map", "iostream", "stdio.h", "stdlib.h", "math.h", "time.h", "chrono", "algorithm"):
        ahead += ["-include", h]
    cmd = ["g++", "-std=c++17", "-O2", "-w", "-fPIC", "-shared", "-I" + build.INCLUDE, "-I" + os.path.join(build.INCLUDE, "tiramisu", "shim"),
           "-I" + source] + ahead + ["-include", entry, "-Dmain=tiramisu_wrapper_main", "-o", library(name), "-x", "c++", "-", "-x", "none"] + objects + \
          ["-L" + build.PKG, "-ltiramisu_hip_wrappers", "-Wl,-rpath,$ORIGIN/" + os.path.relpath(build.PKG, bdir)]
    r = subprocess.run(cmd, input=text, text=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if r.returncode != 0:
        raise RuntimeError("wrapper of %s failed to compile:\n%s" % (name, r.stdout[-3000:]))


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


# The library LSTM in double precision: the reference publishes figures for it (gpu_lib/README.md:7-14) and
# its configuration.h carries the switch ("#if 1  // Flip to use double precision").  The switch is flipped on
# the way into the compiler -- the header, flipped, and the generator without its include line go through a pipe
# to g++ -- so nothing of the reference is written anywhere; everything else is as for the float build.
def build_lstm_gpu_lib_f64():
    import subprocess
    rel = "benchmarks/DNN/blocks/LSTM/gpu_lib/generator.cpp"
    bdir = os.path.join(HERE, "build")
    work = os.path.join(bdir, "lstm_gpu_lib_f64")
    os.makedirs(work, exist_ok=True)
    src = os.path.join(REFERENCE, rel)
    header = open(os.path.join(os.path.dirname(src), "configuration.h")).read()
    if "#if 1  // Flip to use double precision" not in header:
        raise RuntimeError("the precision switch of the reference's LSTM configuration moved")
    text = header.replace("#if 1  // Flip to use double precision", "#if 0") + "\n" + \
        "".join(line for line in open(src) if '#include "configuration.h"' not in line)
    gen = os.path.join(work, "gen")
    cmd = ["g++", "-std=c++17", "-O1", "-x", "c++", "-", "-I" + build.INCLUDE, "-I" + os.path.join(build.INCLUDE, "tiramisu", "shim"),
           "-I" + os.path.dirname(src), "-o", gen, "-L" + build.PKG, "-ltiramisu", "-Wl,-rpath," + build.PKG]
    done = subprocess.run(cmd, input=text.encode(), stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if done.returncode != 0:
        sys.stderr.write(done.stdout.decode())
        raise RuntimeError("build step failed: the reference's library LSTM in double precision")
    build._run([gen], cwd=work)
    build._run(["g++", "-shared", "-o", library("lstm_gpu_lib_f64"), os.path.join(work, "lstm.o"), "-L" + build.PKG,
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


# The reference's tuned CPU schedules of two benchmark configurations, unchanged, through the oracle's CPU emitter:
#  * benchmarks/linear_algebra/blas/level3/sgemm/cpu/sgemm_generator.cpp (packed B, three-level tiling, separated
#    partial tiles; sizes at run time);
#  * benchmarks/DNN/layers/convolution/direct/cpu/conv_layer_generator_tiramisu.cpp (blocked layouts, a register tile
#    named through a tiramisu::view; its configure.h uses std::sort without <algorithm>, which is forced in here).
#    Its register tile is one temporary buffer shared by the iterations of its parallel loops -- the reference counts
#    on LLVM keeping it in registers -- so the generated code is only right on one thread.
CPU_BENCHMARKS = [("benchmarks/linear_algebra/blas/level3/sgemm/cpu/sgemm_generator.cpp", "sgemm_cpu_tuned", "generated_sgemm.o", ["-I" + os.path.join(REFERENCE, "benchmarks")]),
                  ("benchmarks/DNN/layers/convolution/direct/cpu/conv_layer_generator_tiramisu.cpp", "conv_cpu_tuned", "generated_conv_layer.o", ["-include", "algorithm"])]


def build_cpu_benchmark(rel, stem, obj, extra):
    from oracle import build as oracle_build
    bdir = os.path.join(HERE, "build")
    work = os.path.join(bdir, stem)
    os.makedirs(work, exist_ok=True)
    src = os.path.join(REFERENCE, rel)
    gen = os.path.join(work, "gen")
    cpu_dir = os.path.dirname(oracle_build.CPU_BACKEND)
    build._run(["g++", "-std=c++17", "-O1"] + extra + ["-I" + build.INCLUDE, "-I" + os.path.join(build.INCLUDE, "tiramisu", "shim"),
                "-I" + os.path.dirname(src), "-o", gen, src,
                "-L" + build.PKG, "-ltiramisu", "-Wl,--no-as-needed", "-L" + cpu_dir, "-ltiramisu_cpu_backend", "-Wl,--as-needed",
                "-Wl,-rpath," + build.PKG, "-Wl,-rpath," + cpu_dir])
    build._run([gen], cwd=work)
    build._run(["g++", "-shared", "-fopenmp", "-o", library(stem), os.path.join(work, obj)])


# The reference's own test-suite (tests/test_N.cpp + wrapper_test_N.cpp, both unchanged) through this
# front-end and the oracle's CPU emitter (GPU tests among them with TIRAMISU_FORCE_ARCH=cpu): each wrapper
# fills its inputs, calls the generated function and compares with the expectation its authors wrote.
# Listed: the tests that pass; 179-195, 198, 199 are the tests of the dependence analysis, the legality checks, the
# shifts that repair a fusion and the skewing solvers (the generator itself asserts what each check must answer,
# so building them runs the checks; the wrappers of SUITE_SILENT print nothing).  Not listed, by cause:
# distributed tags, Halide image I/O (not provided by this front-end; test 14, compute_at on a loaded image, among
# them); 27, 130 (compute_bounds: the wrapper hands a 1-element buffer to a 10x10 program), 82, 83, 90 (store_at /
# compute_at programs that the reference's own test list leaves out as well: 83 expects values where its
# consumer's domain has none); 94, 95, 172-174
# (wrapper and generator disagree in the reference itself: expected value 2 against a generated 1, a
# 10-element buffer handed to a 100-iteration loop); 133-140 (a recurrence whose dependent loop the test
# tags parallel: the result depends on thread timing).
SUITE = """01 02 03 04 06 07 08 09 10 11 12 13 16 17 18 19 20 21 22 23 24 25 26 29 30 31 32 33 34 35 36 37 38 39 40 41 42 43 44 45 46 47 48 51 52 53 54 55 56 57 58 59 60 61 62 63 64
65 66 67 68 69 70 71 72 73 74 75 76 77 78 79 80 81 84 86 87 88 89 91 92 97 103 104 105 106 107 108 109 110 111 112 113 114 115 116 117 118 119 120 121 122 123
124 125 126 127 128 129 131 141 142 143 144 145 146 147 148 149 150 151 152 153 154 155 156 157 158 159 161 163 167 168 169 170 171 175
176 177 178 179 180 181 182 183 184 185 186 187 188 189 190 191 192 193 194 195 196 197 198 199""".split()

# wrappers that call the generated function and print nothing: the test is the generator's own assertions
# (196: that the unrolled and vectorized loops with their remainders generate and run)
SUITE_SILENT = ["183", "184", "191", "196"]


# Developer tutorials of the reference that pass the same way (04gpu and 04gpu2 run on the GPU, above; 01's
# wrapper hands an int32 buffer to a uint8 function, 11 and 12 are distributed, 13 accesses a 2-D computation
# with one index -- an error in the reference too).
SUITE_TUTORIALS = ["tutorial_02", "tutorial_03", "tutorial_04A", "tutorial_04B", "tutorial_05", "tutorial_06", "tutorial_07", "tutorial_08",
                   "tutorial_10"]


def suite_sources(n):
    if n.startswith("tutorial_"):
        d = os.path.join(REFERENCE, "tutorials", "developers", n)
        return d, os.path.join(d, n + ".cpp"), os.path.join(d, "wrapper_" + n + ".cpp")
    d = os.path.join(REFERENCE, "tests")
    return d, os.path.join(d, "test_%s.cpp" % n), os.path.join(d, "wrapper_test_%s.cpp" % n)


def suite_program(n):
    return os.path.join(HERE, "build", "suite", n, "wrapper")


def build_suite_test(n):
    import subprocess
    from oracle import build as oracle_build
    work = os.path.join(HERE, "build", "suite", n)
    os.makedirs(os.path.join(work, "build"), exist_ok=True)
    tests, generator_source, wrapper_source = suite_sources(n)
    shim = os.path.join(build.INCLUDE, "tiramisu", "shim")
    cpu_dir = os.path.dirname(oracle_build.CPU_BACKEND)
    gen = os.path.join(work, "gen")
    build._run(["g++", "-std=c++17", "-O0", "-w", "-I" + build.INCLUDE, "-I" + shim, "-I" + tests, "-o", gen, generator_source,
                "-L" + build.PKG, "-ltiramisu", "-Wl,--no-as-needed", "-L" + cpu_dir, "-ltiramisu_cpu_backend", "-Wl,--as-needed",
                "-Wl,-rpath," + build.PKG, "-Wl,-rpath," + cpu_dir])
    for f in os.listdir(os.path.join(work, "build")):
        os.remove(os.path.join(work, "build", f))
    env = dict(os.environ)
    env["TIRAMISU_FORCE_ARCH"] = "cpu"
    r = subprocess.run([gen], cwd=work, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("generator of reference test %s failed:\n%s" % (n, r.stdout[-2000:]))
    objects = [os.path.join(work, "build", f) for f in os.listdir(os.path.join(work, "build")) if f.endswith(".o")]
    build._run(["g++", "-std=c++17", "-O0", "-w", "-fopenmp", "-I" + build.INCLUDE, "-I" + shim, "-I" + tests, "-o", suite_program(n),
                wrapper_source] + objects +
               ["-L" + build.PKG, "-ltiramisu_hip_wrappers", "-ltiramisu", "-Wl,-rpath,$ORIGIN/" + os.path.relpath(build.PKG, work)])


def build_suite(verbose=False):
    from concurrent.futures import ThreadPoolExecutor
    if verbose:
        print("[reference programs] tests/test_N.cpp + wrapper_test_N.cpp: %d tests through the CPU emitter" % len(SUITE), flush=True)
    with ThreadPoolExecutor(8) as pool:
        list(pool.map(build_suite_test, SUITE + SUITE_TUTORIALS))


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
    for rel in BARYON:
        if verbose:
            print("[reference programs]", rel, flush=True)
        build_baryon(rel)
    if os.environ.get("TIRAMISU_BUILD_DIBARYON") == "1":
        for rel in DIBARYON:
            if verbose:
                print("[reference programs]", rel, "(about ten minutes)", flush=True)
            build_dibaryon(rel)
    if verbose:
        print("[reference programs] benchmarks/DNN/blocks/LSTM/gpu_lib/generator.cpp (double precision)", flush=True)
    build_lstm_gpu_lib_f64()
    if verbose:
        print("[reference programs]", LSTM_NAIVE, "(CPU)", flush=True)
    build_lstm_naive()
    for rel, stem, obj, extra in CPU_BENCHMARKS:
        if verbose:
            print("[reference programs]", rel, "(CPU)", flush=True)
        build_cpu_benchmark(rel, stem, obj, extra)
    build_suite(verbose)
    return True


if __name__ == "__main__":
    build_all(verbose=True)
