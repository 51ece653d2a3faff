"""Builds the oracle's native parts (test infrastructure; nothing in the product imports this).

* oracle/cpu_backend/libtiramisu_cpu_backend.so -- the CPU back-end restatement; linking it into
  a generator registers the arch_cpu target.
* <program dir>/build/lib<name>_cpu.so -- every Tiramisu program compiled for the host: programs
  with their own CPU schedule are built with -DTIRAMISU_TARGET_CPU, the others are forced onto
  the CPU back-end with TIRAMISU_FORCE_ARCH=cpu (GPU-mapped loops then run serially).
"""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from tiramisu_amd import build as product_build  # noqa: E402  (compiler library and include paths only)

ORACLE = os.path.join(ROOT, "oracle")
CPU_BACKEND = os.path.join(ORACLE, "cpu_backend", "libtiramisu_cpu_backend.so")


def _run(cmd, cwd=None, env=None):
    r = subprocess.run(cmd, cwd=cwd, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write("command failed: %s\n%s\n" % (" ".join(cmd), r.stdout))
        raise RuntimeError("oracle build step failed")
    return r.stdout


def build_cpu_backend():
    _run(["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-I" + product_build.INCLUDE, "-o", CPU_BACKEND,
          os.path.join(ORACLE, "cpu_backend", "cpu_emit.cpp"), "-L" + product_build.PKG, "-ltiramisu",
          "-Wl,-rpath," + product_build.PKG])


def cpu_program_library(directory, name):
    return os.path.join(directory, "build", "lib%s_cpu.so" % name)


def build_cpu_program(source):
    directory = os.path.dirname(os.path.abspath(source))
    stem = os.path.splitext(os.path.basename(source))[0]
    bdir = os.path.join(directory, "build")
    os.makedirs(bdir, exist_ok=True)
    text = open(source).read()
    if "NO_CPU_VARIANT" in text:
        return
    own_schedule = "TIRAMISU_TARGET_CPU" in text
    gen = os.path.join(bdir, "gen_cpu_" + stem)
    _run(["g++", "-std=c++17", "-O1", "-I" + product_build.INCLUDE, "-I" + directory] +
         (["-DTIRAMISU_TARGET_CPU"] if own_schedule else []) +
         ["-o", gen, source, "-L" + product_build.PKG, "-ltiramisu", "-Wl,--no-as-needed",
          "-L" + os.path.dirname(CPU_BACKEND), "-ltiramisu_cpu_backend", "-Wl,--as-needed",
          "-Wl,-rpath," + product_build.PKG, "-Wl,-rpath," + os.path.dirname(CPU_BACKEND)])
    env = dict(os.environ)
    env["TIRAMISU_FORCE_ARCH"] = "cpu"
    before = {f: os.path.getmtime(os.path.join(bdir, f)) for f in os.listdir(bdir) if f.endswith("_cpu.o")}
    _run([gen], cwd=directory, env=env)
    for obj in os.listdir(bdir):
        if not obj.endswith("_cpu.o"):
            continue
        if obj in before and os.path.getmtime(os.path.join(bdir, obj)) <= before[obj]:
            continue
        name = obj[:-2]
        if name.startswith("generated_fct_"):
            name = name[len("generated_fct_"):]
        _run(["g++", "-shared", "-fopenmp", "-o", os.path.join(bdir, "lib%s.so" % name), os.path.join(bdir, obj)])


def build_all(force=True, verbose=False):
    build_cpu_backend()
    for src in product_build.program_sources():
        if verbose:
            print("[oracle build] cpu variant of", os.path.relpath(src, ROOT), flush=True)
        build_cpu_program(src)


if __name__ == "__main__":
    build_all(verbose=True)
