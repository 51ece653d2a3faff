"""The runtime C ABI: the shared library loads without a GPU and exports every entry point that
include/tiramisu_hip_wrappers.h declares (no compute calls here)."""
import ctypes
import os
import re

from tiramisu_amd import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tiramisu_hip_wrappers.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tiramisu_hip_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_reference_shims():
    names = declared_symbols()
    for n in ["tiramisu_hip_malloc", "tiramisu_hip_free", "tiramisu_hip_memcpy_to_device",
              "tiramisu_hip_memcpy_to_host", "tiramisu_hip_memcpy_to_symbol", "tiramisu_hip_sgemm",
              "tiramisu_hip_dgemm", "tiramisu_hip_stream_synchronize", "tiramisu_hip_module_load",
              "tiramisu_hip_launch"]:
        assert n in names


def test_library_exports_every_declared_symbol():
    path = build.wrappers_library()
    assert os.path.exists(path), "run __graft_entry__.build() first"
    lib = ctypes.CDLL(path)
    for n in declared_symbols():
        assert hasattr(lib, n), n


def test_compiler_library_loads():
    assert os.path.exists(build.compiler_library())
    ctypes.CDLL(build.compiler_library())


def test_generated_program_exports_its_function():
    wr = ctypes.CDLL(build.wrappers_library(), mode=ctypes.RTLD_GLOBAL)
    assert wr is not None
    lib = ctypes.CDLL(build.program_library(os.path.join(ROOT, "tests", "programs"), "gemm_gpu_tile"))
    assert hasattr(lib, "gemm_gpu_tile")
