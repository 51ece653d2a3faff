"""The CMake build boundary (CMakeLists.txt + configure.cmake at the repository root, the counterpart of
the reference's USE_GPU / cuda_wrapper / set_obj machinery, CMakeLists.txt:24-34, :229-271 and
configure.cmake:5-19 there): configuring and building with cmake gives the same two libraries as
tiramisu_amd/build.py, the cmake-built runtime exports exactly the C ABI the header declares, and --
where a Tiramisu source tree is at hand -- the reference's GPU tests are registered with the `hip`
label and one of them (generator + wrapper, unchanged) builds through the `new_test` helper.
Nothing here needs a GPU: hipcc cross-compiles."""
import os
import re
import shutil
import subprocess

import pytest

from test_abi import declared_symbols

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = os.environ.get("TIRAMISU_REFERENCE_TREE", "/root/reference")


def run(cmd, **kw):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    assert r.returncode == 0, "%s failed:\n%s" % (" ".join(cmd), r.stdout[-3000:])
    return r.stdout


def exported(lib):
    out = run(["nm", "-D", "--defined-only", lib])
    return sorted(set(re.findall(r"\b[TW] (tiramisu_hip_[a-z_0-9]+)$", out, re.M)))


@pytest.fixture(scope="module")
def cmake_build():
    if shutil.which("cmake") is None:
        pytest.skip("cmake is not installed")
    from tiramisu_amd import build
    return build.build_cmake(REFERENCE)      # configures, then builds what is out of date


def test_cmake_builds_both_libraries(cmake_build):
    bdir, _ = cmake_build
    assert os.path.exists(os.path.join(bdir, "libtiramisu.so"))
    assert os.path.exists(os.path.join(bdir, "libtiramisu_hip_wrappers.so"))


def test_cmake_runtime_exports_the_declared_abi(cmake_build):
    bdir, _ = cmake_build
    from tiramisu_amd import build
    mine = exported(os.path.join(bdir, "libtiramisu_hip_wrappers.so"))
    assert mine == declared_symbols()
    assert mine == exported(build.wrappers_library())       # the library build.py makes exports the same set


def test_installed_tree_is_self_contained(cmake_build, tmp_path):
    """cmake --install: lib/, include/ and share/tiramisu/kernels.  A generator compiled against the installed headers
    and library alone generates a GPU function whose device code (kernel headers included by file name) was compiled
    against the installed kernel headers, found relative to the installed library -- not through a path into this
    source tree -- and whose host glue was compiled against the installed tiramisu_hip_wrappers.h."""
    import json
    bdir, _ = cmake_build
    prefix = os.path.join(str(tmp_path), "prefix")
    run(["cmake", "--install", bdir, "--prefix", prefix])
    for rel in ("lib/libtiramisu.so", "lib/libtiramisu_hip_wrappers.so", "include/tiramisu/tiramisu.h",
                "include/tiramisu_hip_wrappers.h", "share/tiramisu/kernels/gemm_mfma.hip.h",
                "share/tiramisu/kernels/stencil2d_regs.hip.h", "share/tiramisu/kernels/wave_reduce.hip.h"):
        assert os.path.exists(os.path.join(prefix, rel)), rel
    work = os.path.join(str(tmp_path), "work")
    os.makedirs(os.path.join(work, "build"))
    gen = os.path.join(work, "gen")
    run(["g++", "-std=c++17", "-O1", "-I" + os.path.join(prefix, "include"), "-o", gen,
         os.path.join(ROOT, "tiramisu_amd", "programs", "sgemm.cpp"), "-L" + os.path.join(prefix, "lib"), "-ltiramisu",
         "-Wl,-rpath," + os.path.join(prefix, "lib")])
    env = {k: v for k, v in os.environ.items() if k not in ("TIRAMISU_AMD_KERNEL_DIR", "TIRAMISU_AMD_INCLUDE")}
    subprocess.run([gen], cwd=work, env=env, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    manifest = json.load(open(os.path.join(work, "build", "sgemm_1024x1024x1024.o.json")))
    assert os.path.realpath(manifest["kernel_headers"]) == os.path.realpath(os.path.join(prefix, "share", "tiramisu", "kernels"))
    text = open(os.path.join(work, "build", "sgemm_1024x1024x1024.o.hip")).read()
    assert '#include "gemm_mfma.hip.h"' in text
    assert ROOT not in text                    # no path into the source tree in the generated device code
    assert os.path.getsize(os.path.join(work, "build", "sgemm_1024x1024x1024.o.hsaco")) > 0


def test_reference_gpu_tests_are_registered_with_the_hip_label(cmake_build):
    bdir, with_tests = cmake_build
    if not with_tests:
        pytest.skip("no Tiramisu source tree at " + REFERENCE)
    listing = run(["ctest", "--test-dir", bdir, "-N", "-L", "hip"])
    for n in ("17", "18", "19", "162", "164", "165", "166", "167", "168", "169", "170", "171", "197"):
        assert re.search(r"Test +#\d+: %s$" % n, listing, re.M), n
        assert re.search(r"Test +#\d+: %s_build$" % n, listing, re.M), n


def test_new_test_helper_builds_a_reference_gpu_test(cmake_build):
    """set_obj / build_g / build_w: the generator of reference test 167 is compiled and run (it calls
    hipcc for the gfx950 code object), and the unchanged wrapper links against the one object it wrote
    plus hip_wrapper."""
    bdir, with_tests = cmake_build
    if not with_tests:
        pytest.skip("no Tiramisu source tree at " + REFERENCE)
    assert os.path.exists(os.path.join(bdir, "tests", "build", "generated_fct_test_167.o"))
    assert os.path.exists(os.path.join(bdir, "test_167"))
    needed = run(["readelf", "-d", os.path.join(bdir, "test_167")])
    assert "libtiramisu_hip_wrappers.so" in needed


def hip_test_ids():
    from tiramisu_amd import build
    return list(build.CMAKE_HIP_TESTS)


@pytest.mark.gpu
@pytest.mark.parametrize("n", hip_test_ids())
def test_cmake_built_reference_gpu_test_passes(n):
    """What `ctest -L hip` runs: the executable test_<n> that the CMake build linked from the reference's
    wrapper_test_<n>.cpp, the object its generator wrote and hip_wrapper.  The wrapper computes its own
    expectation and exits with status 1 on a mismatch (the reference's compare_buffers)."""
    from tiramisu_amd import build
    exe = os.path.join(build.CMAKE_BUILD, "test_" + n)
    if not os.path.exists(exe):
        pytest.skip("the CMake build has not produced test_%s (no Tiramisu source tree when it ran)" % n)
    print("running cmake-built test_" + n, flush=True)
    r = subprocess.run([exe], cwd=os.path.join(build.CMAKE_BUILD, "tests"), stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True, timeout=100)
    assert r.returncode == 0, r.stdout[-2000:]
