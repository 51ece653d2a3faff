"""Runs one of the reference's Python tutorials (python_bindings/tutorials/*.py, read where it lies, unchanged) against
this build's `tiramisu` module: usage  run_python_tutorial.py <path of the tutorial>  from the directory that is
to receive the generated files.  The tutorials generate CPU code; this package ships no CPU back-end, so the test
harness registers the oracle's restatement of it (loading the library is what registers it) -- test infrastructure,
not a product path."""
import ctypes
import os
import runpy
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "tiramisu_amd", "python"))
sys.path.insert(0, ROOT)

import tiramisu  # noqa: E402,F401  (loads the compiler library the CPU emitter registers with)
from oracle import build as oracle_build  # noqa: E402

ctypes.CDLL(oracle_build.CPU_BACKEND, mode=ctypes.RTLD_GLOBAL)
runpy.run_path(sys.argv[1], run_name="__main__")
