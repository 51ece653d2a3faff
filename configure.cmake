# Build options of the Tiramisu HIP back-end.  Mirrors the reference's configure.cmake
# (its USE_GPU / WITH_TESTS / DEBUG_LEVEL options, configure.cmake:5-19): a Tiramisu tree that
# adopts this back-end adds the USE_HIP block next to USE_GPU and keeps everything else.

option(USE_HIP "Build the HIP back-end runtime (hip_wrapper) for AMD GPUs" ON)

# Device compiler and target of the kernels the back-end emits.  HIPCC_PATH is also the default
# the compiler library falls back to when the environment variable of the same name is unset
# (the reference bakes NVCC_PATH in the same way, CMakeLists.txt:26).
set(HIPCC_PATH "/opt/rocm/bin/hipcc" CACHE FILEPATH "hipcc used for the runtime library and by generated-code compilation")
set(TIRAMISU_HIP_ARCH "gfx950" CACHE STRING "--offload-arch of the runtime library and default target of emitted kernels")

# isl: the library is linked by file name because images ship the runtime library without the
# development symlink (the reference points ISL_LIB_DIRECTORY at its vendored build instead).
set(ISL_LIBRARY "-l:libisl.so.23" CACHE STRING "Linker argument for isl")

option(WITH_TESTS "Register the reference's GPU tests (generator + wrapper, unchanged) with the [hip] tag" OFF)
# Root of a Tiramisu source tree whose tests/test_N.cpp and tests/wrapper_test_N.cpp are compiled in
# place when WITH_TESTS is on.
set(TIRAMISU_REFERENCE_DIR "" CACHE PATH "Tiramisu source tree holding tests/ and tutorials/")

option(WITH_PYTHON_BINDINGS "Build the pybind11 module of the Python front-end" OFF)

set(DEBUG_LEVEL 0 CACHE STRING "Debug level value")
