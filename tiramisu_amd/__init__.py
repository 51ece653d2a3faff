"""MI355X-native GPU back-end for the Tiramisu polyhedral compiler.

The product is native code: ``libtiramisu.so`` (the C++ front-end and the HIP/host emitters) and
``libtiramisu_hip_wrappers.so`` (the runtime C ABI).  The Python modules only build those
libraries (``build``) and call compiled Tiramisu functions through their C ABI (``runtime``).
"""
from . import build, runtime  # noqa: F401
