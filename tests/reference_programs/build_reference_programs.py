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
]


def library(name):
    return os.path.join(HERE, "build", "lib%s.so" % name)


def build_all(verbose=False):
    if not os.path.isdir(REFERENCE):
        if verbose:
            print("[reference programs] %s is absent: nothing built" % REFERENCE)
        return False
    for rel, defines, name in PROGRAMS:
        if verbose:
            print("[reference programs]", rel, flush=True)
        build.build_program(os.path.join(REFERENCE, rel), defines=defines, directory=HERE, shim_headers=True)
    return True


if __name__ == "__main__":
    build_all(verbose=True)
