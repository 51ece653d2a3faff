"""The stencil kernel's loads and stores, enumerated on the host.

tests/host_models/stencil_address_model.cpp compiles kernels/stencil2d_regs.hip.h itself as plain C++ (its
host-model form: every access to global memory is recorded instead of performed) and runs every workgroup and
thread of every launch that the emitter's plan (csrc/stencil_plan.h) makes for plane sizes 5 ... 300 (every
residue mod 4, square and not), 1 ... 13 steps per launch and the four kernel modes: loads inside their buffer
and aligned, every cell a launch owes written exactly once and nothing else, whole time loops ending with the
right steps in the right planes.  The second test breaks the kernel's indexing in a copy and expects the model
to say so: a model that cannot fail pins nothing.
"""
import os
import shutil
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MODEL = os.path.join(ROOT, "tests", "host_models", "stencil_address_model.cpp")


def build_model(source, out):
    subprocess.run(["g++", "-std=c++17", "-O2", "-Wno-unknown-pragmas", "-o", out, source], check=True)


def test_every_load_and_store_of_the_stencil_kernel_is_in_bounds_and_owed(tmp_path):
    exe = str(tmp_path / "model")
    build_model(MODEL, exe)
    r = subprocess.run([exe], stdout=subprocess.PIPE, text=True)
    print(r.stdout[-2000:])
    assert r.returncode == 0, r.stdout[-2000:]
    assert " 0 failure(s)" in r.stdout


def test_the_model_reports_broken_indexing(tmp_path):
    """Three one-token mistakes in a copy of the kernel: a tile one row too tall, a strip one lane too wide, a
    region shifted by one quad.  Each must be reported."""
    tree = tmp_path / "copy"
    (tree / "tests" / "host_models").mkdir(parents=True)
    (tree / "tiramisu_amd" / "csrc" / "kernels").mkdir(parents=True)
    shutil.copy(MODEL, tree / "tests" / "host_models")
    shutil.copy(os.path.join(ROOT, "tiramisu_amd", "csrc", "stencil_plan.h"), tree / "tiramisu_amd" / "csrc")
    kernels = os.path.join(ROOT, "tiramisu_amd", "csrc", "kernels")
    for h in ("stencil2d_regs.hip.h", "target_gfx950.h"):
        shutil.copy(os.path.join(kernels, h), tree / "tiramisu_amd" / "csrc" / "kernels")
    original = open(os.path.join(kernels, "stencil2d_regs.hip.h")).read()
    mistakes = [("gy >= row_end) continue;", "gy > row_end) continue;", ["5", "60", "5"]),
                ("4 * lane < ST_HX + ST_TW)", "4 * lane <= ST_HX + ST_TW)", ["290", "300", "3"]),
                ("const int gx = ox - ST_HX + 4 * lane;", "const int gx = ox - ST_HX + 4 * lane + 4;", ["5", "40", "3"])]
    for old, new, sweep in mistakes:
        assert original.count(old) == 1, old
        (tree / "tiramisu_amd" / "csrc" / "kernels" / "stencil2d_regs.hip.h").write_text(original.replace(old, new))
        exe = str(tmp_path / "broken")
        build_model(str(tree / "tests" / "host_models" / "stencil_address_model.cpp"), exe)
        r = subprocess.run([exe] + sweep, stdout=subprocess.PIPE, text=True)
        assert r.returncode != 0 and "FAIL" in r.stdout, "the model accepted: " + new
