"""Build steps of the Tiramisu HIP back-end.

Three kinds of artefacts, all in-tree so that they travel to the GPU machine:

* ``tiramisu_amd/libtiramisu.so``              the compiler (front-end over isl, AST lowering,
                                               HIP + host-glue emitters), plain C++ (g++);
* ``tiramisu_amd/libtiramisu_hip_wrappers.so`` the runtime C ABI (hipcc, gfx950);
* ``<dir>/build/lib<program>.so``              one shared library per Tiramisu program: the
                                               generator is compiled and run here (it calls hipcc
                                               to produce the gfx950 code object), and the host
                                               object it writes is linked against the runtime.

Nothing here needs a GPU: hipcc cross-compiles for gfx950.
"""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "tiramisu_amd")
CSRC = os.path.join(PKG, "csrc")
INCLUDE = os.path.join(ROOT, "include")
HIPCC = os.environ.get("HIPCC_PATH", "/opt/rocm/bin/hipcc")
ISL = "-l:libisl.so.23"
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

COMPILER_SOURCES = ["expr.cpp", "core.cpp", "astgen.cpp", "c_print.cpp", "hip_backend.cpp", "evaluator.cpp",
                    "recognize.cpp", "dependences.cpp"]

PROGRAM_DIRS = [os.path.join(PKG, "programs"), os.path.join(ROOT, "tests", "programs")]


def _run(cmd, cwd=None, quiet=True):
    r = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write("command failed: %s\n%s\n" % (" ".join(cmd), r.stdout))
        raise RuntimeError("build step failed: " + " ".join(cmd[:3]))
    if not quiet and r.stdout.strip():
        print(r.stdout)
    return r.stdout


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources if os.path.exists(s))


def compiler_library():
    return os.path.join(PKG, "libtiramisu.so")


def wrappers_library():
    return os.path.join(PKG, "libtiramisu_hip_wrappers.so")


def build_compiler(force=True):
    srcs = [os.path.join(CSRC, s) for s in COMPILER_SOURCES]
    deps = srcs + [os.path.join(CSRC, h) for h in os.listdir(CSRC) if h.endswith(".h")] + \
        [os.path.join(INCLUDE, "tiramisu", h) for h in os.listdir(os.path.join(INCLUDE, "tiramisu"))]
    kdir = os.path.join(CSRC, "kernels")
    deps += [os.path.join(kdir, h) for h in os.listdir(kdir)]
    out = compiler_library()
    if not force and _newer(out, deps):
        return out
    _run(["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-I" + INCLUDE,
          '-DTIRAMISU_AMD_INCLUDE_DIR="%s"' % INCLUDE,
          '-DTIRAMISU_AMD_KERNEL_DIR="%s"' % kdir,
          "-o", out] + srcs + [ISL])
    return out


def build_wrappers(force=True):
    src = os.path.join(CSRC, "hip_wrappers.hip")
    kdir = os.path.join(CSRC, "kernels")
    deps = [src, os.path.join(INCLUDE, "tiramisu_hip_wrappers.h")] + \
        [os.path.join(kdir, h) for h in os.listdir(kdir)]
    out = wrappers_library()
    if not force and _newer(out, deps):
        return out
    _run([HIPCC] + HIP_FLAGS + ["-fPIC", "-shared", "-o", out, src])
    return out


def program_library(directory, name):
    return os.path.join(directory, "build", "lib%s.so" % name)


def build_program(source, force=True, extra_objects=(), defines=(), directory=None, shim_headers=False):
    """Compile and run the generator ``source`` (a Tiramisu program), then link every host
    object it wrote (build/<x>.o) into build/lib<x>.so -- next to the source, or under
    ``directory`` when the source lies in a tree that must not be written to.  ``shim_headers``
    adds the stand-ins of include/tiramisu/shim (Halide.h, isl/*.h) to the include path, for
    programs written against the reference's include set."""
    source_dir = os.path.dirname(os.path.abspath(source))
    directory = os.path.abspath(directory) if directory else source_dir
    stem = os.path.splitext(os.path.basename(source))[0]
    bdir = os.path.join(directory, "build")
    os.makedirs(bdir, exist_ok=True)
    gen = os.path.join(bdir, "gen_" + stem)
    stamp = os.path.join(bdir, stem + ".stamp")
    if not force and _newer(stamp, [source, compiler_library(), wrappers_library()]):
        return
    before = {f: os.path.getmtime(os.path.join(bdir, f)) for f in os.listdir(bdir) if f.endswith(".o")}
    shim = ["-I" + os.path.join(INCLUDE, "tiramisu", "shim")] if shim_headers else []
    _run(["g++", "-std=c++17", "-O1", "-I" + INCLUDE, "-I" + source_dir] + shim + ["-D" + d for d in defines] +
         ["-o", gen, source] + list(extra_objects) +
         ["-L" + PKG, "-ltiramisu", "-Wl,-rpath," + PKG])
    env_out = _run([gen], cwd=directory)
    produced = [f for f in os.listdir(bdir) if f.endswith(".o") and
                (f not in before or os.path.getmtime(os.path.join(bdir, f)) > before[f])]
    for obj in produced:
        name = obj[:-2]
        if name.startswith("generated_fct_"):
            name = name[len("generated_fct_"):]
        lib = os.path.join(bdir, "lib%s.so" % name)
        _run(["g++", "-shared", "-o", lib, os.path.join(bdir, obj), "-L" + PKG, "-ltiramisu_hip_wrappers",
              "-Wl,-rpath,$ORIGIN/" + os.path.relpath(PKG, bdir)])
    with open(stamp, "w") as f:
        f.write(env_out)
    return produced


def program_sources():
    out = []
    for d in PROGRAM_DIRS:
        if os.path.isdir(d):
            out += sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(".cpp"))
    return out


WRAPPER_DIR = os.path.join(ROOT, "tests", "wrappers")


def wrapper_library(name):
    return os.path.join(WRAPPER_DIR, "build", "lib%s.so" % name)


def build_wrapper_program(source):
    """Link a C++ wrapper program (main() + Halide::Buffer arguments, the reference's
    tests/wrapper_test_*.cpp style) with the generated object named in its first
    ``// links: <dir>/<object>`` line into a shared library whose entry point is
    ``tiramisu_wrapper_main`` (the program's main), so that a test can run it in-process."""
    stem = os.path.splitext(os.path.basename(source))[0]
    objects = []
    for line in open(source):
        if line.startswith("// links:"):
            objects += [os.path.join(ROOT, o) for o in line[len("// links:"):].split()]
    os.makedirs(os.path.join(WRAPPER_DIR, "build"), exist_ok=True)
    entry = os.path.join(WRAPPER_DIR, "build", "entry.h")
    with open(entry, "w") as f:
        f.write('extern "C" int tiramisu_wrapper_main(int, char **);\n')
    _run(["g++", "-std=c++17", "-O1", "-fPIC", "-shared", "-I" + INCLUDE, "-I" + os.path.join(INCLUDE, "tiramisu", "shim"),
          "-include", entry, "-Dmain=tiramisu_wrapper_main", "-o", wrapper_library(stem), source] + objects +
         ["-L" + PKG, "-ltiramisu_hip_wrappers", "-Wl,-rpath,$ORIGIN/" + os.path.relpath(PKG, os.path.join(WRAPPER_DIR, "build"))])


PYTHON_PACKAGE = os.path.join(PKG, "python", "tiramisu")
PYTHON_PROGRAMS = os.path.join(ROOT, "tests", "python_programs")


def python_module():
    import sysconfig
    return os.path.join(PYTHON_PACKAGE, "tiramisu" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_python_module():
    """The pybind11 extension behind ``from tiramisu import *`` (tiramisu_amd/python/tiramisu)."""
    import sysconfig
    import pybind11
    _run(["g++", "-std=c++17", "-O1", "-fPIC", "-shared", "-fvisibility=hidden", "-I" + INCLUDE, "-I" + pybind11.get_include(),
          "-I" + sysconfig.get_paths()["include"], "-o", python_module(), os.path.join(CSRC, "python_module.cpp"),
          "-L" + PKG, "-ltiramisu", "-Wl,-rpath,$ORIGIN/../.."])
    return python_module()


def build_python_programs(verbose=False):
    """Run the Tiramisu programs written in Python (tests/python_programs/*.py): each generates its
    object and links lib<function>.so under tests/python_programs/build/."""
    if not os.path.isdir(PYTHON_PROGRAMS):
        return
    for f in sorted(os.listdir(PYTHON_PROGRAMS)):
        if f.endswith(".py"):
            if verbose:
                print("[build] python program", f, flush=True)
            _run([sys.executable, os.path.join(PYTHON_PROGRAMS, f)])


CMAKE_BUILD = os.path.join(ROOT, "build", "cmake")
CMAKE_HIP_TESTS = ("17", "18", "19", "162", "164", "165", "166", "167", "168", "169", "170", "171", "197")


def build_cmake(reference_tree=None, verbose=False):
    """The same two libraries through the CMake build (CMakeLists.txt + configure.cmake at the root), into
    build/cmake; with a Tiramisu source tree at hand also the reference's GPU tests that the build
    registers under the `hip` label (generator and wrapper unchanged, executables build/cmake/test_<n>).
    Returns (build directory, whether the tests were built)."""
    import shutil
    if shutil.which("cmake") is None:
        raise RuntimeError("cmake is not installed")
    with_tests = bool(reference_tree) and os.path.isdir(os.path.join(reference_tree, "tests"))
    os.makedirs(CMAKE_BUILD, exist_ok=True)
    cfg = ["cmake", "-S", ROOT, "-B", CMAKE_BUILD, "-DUSE_HIP=ON", "-DWITH_TESTS=" + ("ON" if with_tests else "OFF")]
    if with_tests:
        cfg.append("-DTIRAMISU_REFERENCE_DIR=" + reference_tree)
    _run(cfg)
    if verbose:
        print("[build] cmake --build", os.path.relpath(CMAKE_BUILD, ROOT), flush=True)
    _run(["cmake", "--build", CMAKE_BUILD, "-j8"])
    if with_tests:
        _run(["cmake", "--build", CMAKE_BUILD, "-j8", "--target"] + ["test_" + n for n in CMAKE_HIP_TESTS])
    return CMAKE_BUILD, with_tests


def build_all(force=True, verbose=False):
    build_compiler(force)
    build_wrappers(force)
    build_python_module()
    build_python_programs(verbose)
    for src in program_sources():
        if "CPU_ONLY_PROGRAM" in open(src).read():
            continue  # needs the CPU back-end, which lives with the oracle
        if verbose:
            print("[build] program", os.path.relpath(src, ROOT), flush=True)
        build_program(src, force)
    if os.path.isdir(WRAPPER_DIR):
        for f in sorted(os.listdir(WRAPPER_DIR)):
            if f.endswith(".cpp"):
                build_wrapper_program(os.path.join(WRAPPER_DIR, f))
    # the compiled tuners (they drive the C++ evaluator on the GPU machine; compiling them needs none)
    from . import autotune
    for f in sorted(os.listdir(autotune.TUNING)):
        if f.endswith(".cpp"):
            autotune.build_tuner(f[:-4])


if __name__ == "__main__":
    build_all(force="--force" in sys.argv, verbose=True)
