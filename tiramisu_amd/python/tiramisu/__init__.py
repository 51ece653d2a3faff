"""The Tiramisu front-end from Python (module layout of the reference's python_bindings package:
``from tiramisu import *``), bound to this build's compiler library and HIP back-end.

``pycodegen`` generates code like ``codegen`` and then makes the generated function callable from
Python, as the reference does by building a Cython extension around the object file
(python_bindings/src/PyCodegen.cpp:31-58): here the object is linked into a shared library next
to it and a module named after the function is registered, so that

    pycodegen([b_A, b_B, b_C], "build/matmul.o", True)
    import matmul
    matmul.matmul(A, B, C)          # numpy arrays (host buffers) or tiramisu_amd.runtime.Buffer

works.  Build the extension with ``tiramisu_amd.build.build_python_module()``."""
import os
import subprocess
import sys
import types

from .tiramisu import *          # noqa: F401,F403
from . import tiramisu as _ext

_HERE = os.path.dirname(os.path.abspath(__file__))
_PKG = os.path.dirname(os.path.dirname(_HERE))      # tiramisu_amd/


def pycodegen(arguments, obj_filename, gen_gpu=True, *unused, _function=None):
    """Generate ``obj_filename`` for the implicit function, link it into ``lib<function>.so`` next
    to it and register a module ``<function>`` whose attribute ``<function>`` runs the code."""
    if _function is not None:
        _function.codegen(arguments, obj_filename, bool(gen_gpu), False)
    elif isinstance(gen_gpu, _ext.hardware_architecture_t):
        _ext.codegen(arguments, obj_filename, gen_gpu)
    else:
        _ext.codegen(arguments, obj_filename, bool(gen_gpu))
    name = (_function or _ext.get_implicit_function()).get_name()
    directory = os.path.dirname(os.path.abspath(obj_filename))
    library = os.path.join(directory, "lib%s.so" % name)
    for_gpu = gen_gpu != _ext.hardware_architecture_t.arch_cpu if isinstance(gen_gpu, _ext.hardware_architecture_t) else bool(gen_gpu)
    if for_gpu:
        link = ["-L" + _PKG, "-ltiramisu_hip_wrappers", "-Wl,-rpath," + _PKG]
    else:
        link = ["-fopenmp"]         # an object of a CPU back-end (none ships with this package; one can be registered)
    subprocess.run(["g++", "-shared", "-o", library, os.path.abspath(obj_filename)] + link, check=True)
    sys.path.insert(0, os.path.dirname(_PKG))
    try:
        from tiramisu_amd import runtime
    finally:
        sys.path.pop(0)
    module = types.ModuleType(name)
    module.__file__ = library
    setattr(module, name, runtime.Program(library, name, needs_gpu_runtime=for_gpu))
    sys.modules[name] = module
    return module


def _function_pycodegen(self, arguments, obj_filename, gen_gpu=True):
    """``function.pycodegen`` of the reference's bindings (python_bindings/tiramisu.pyi:309): pycodegen for a
    function object instead of the implicit one."""
    return pycodegen(arguments, obj_filename, gen_gpu, _function=self)


_ext.function.pycodegen = _function_pycodegen
