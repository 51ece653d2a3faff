"""C++ wrapper programs in the reference's style (Halide::Buffer arguments built with the
stand-in of include/tiramisu/shim/Halide.h, helpers of include/tiramisu/utils.h), linked against
generated objects and run in-process: what a user of the reference does with a generated
function, end to end, without Python buffers in between."""
import ctypes
import os

import pytest

from tiramisu_amd import build, runtime

WRAPPERS = ["wrapper_gemm_gpu_tile", "wrapper_taps_in_constant_memory"]


@pytest.mark.parametrize("name", WRAPPERS)
def test_wrapper_library_exports_its_entry_point(name):
    path = build.wrapper_library(name)
    assert os.path.exists(path), "run __graft_entry__.build() first"
    runtime.wrappers()   # the runtime ABI must be loaded first (global symbols)
    lib = ctypes.CDLL(path)
    assert hasattr(lib, "tiramisu_wrapper_main")


@pytest.mark.gpu
@pytest.mark.parametrize("name", WRAPPERS)
def test_wrapper_program_passes(name):
    # the wrapper compares with its own nested-loop reference and ends the process with status 1
    # on a mismatch (the reference's compare_buffers does); 0 means it passed
    runtime.wrappers()
    lib = ctypes.CDLL(build.wrapper_library(name))
    lib.tiramisu_wrapper_main.restype = ctypes.c_int
    lib.tiramisu_wrapper_main.argtypes = [ctypes.c_int, ctypes.c_void_p]
    assert lib.tiramisu_wrapper_main(0, None) == 0
