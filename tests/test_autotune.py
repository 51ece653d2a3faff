"""Host-side pieces of tiramisu_amd.autotune (knob combinations, argument construction from the
back-end's description of a function) and of the argument check in runtime.Program.  Timing runs
need a GPU and a code-generation pass per variant, so they are not part of the test suite."""
import json
import os

import numpy as np
import pytest

from tiramisu_amd import autotune, runtime


def test_knob_combinations():
    got = list(autotune.variants(["A=1,2", "B=x"]))
    assert got == [{"A": "1", "B": "x"}, {"A": "2", "B": "x"}]
    assert list(autotune.variants([])) == [{}]


def test_manifest_describes_arguments_and_kernels(product_programs_dir):
    m = json.load(open(os.path.join(product_programs_dir, "build", "sgemm_1024x1024x1024.o.json")))
    assert m["function"] == "sgemm_1024x1024x1024"
    assert [(a["name"], a["type"], a["kind"], a["memory"], a["shape"]) for a in m["arguments"]] == [
        ("b_scal", "float", "input", "host", [2]), ("b_A", "float", "input", "device", [1024, 1024]),
        ("b_B", "float", "input", "device", [1024, 1024]), ("b_C", "float", "output", "device", [1024, 1024])]
    assert len(m["kernels"]) == 1 and m["kernels"][0]["how"].startswith("mfma-contraction")
    lib = os.path.join(product_programs_dir, "build", "libsgemm_1024x1024x1024.so")
    assert runtime.manifest_of(lib, "sgemm_1024x1024x1024") == m


def test_run_time_extents_are_reported(programs_dir):
    m = json.load(open(os.path.join(programs_dir, "build", "sgemm_runtime_sizes.o.json")))
    assert m["arguments"][2]["shape"] == ["M", "K"]
    with pytest.raises(SystemExit):
        autotune.make_arguments(m, seed=0)


class FakeProgram(runtime.Program):
    def __init__(self, manifest):
        self.manifest, self.name = manifest, manifest["function"]


def test_arguments_are_checked_before_the_call(product_programs_dir):
    m = json.load(open(os.path.join(product_programs_dir, "build", "sgemm_1024x1024x1024.o.json")))
    p = FakeProgram(m)
    scal = runtime.Buffer.from_numpy(np.zeros(2, np.float32))
    dev = lambda shape, dtype=np.float32: runtime.Buffer.from_device(4096, shape, dtype)
    p.check([scal, dev((1024, 1024)), dev((1024, 1024)), dev((1024, 1024))])
    with pytest.raises(ValueError, match="takes 4 buffers"):
        p.check([scal, dev((1024, 1024))])
    with pytest.raises(ValueError, match="shape"):
        p.check([scal, dev((1024, 512)), dev((1024, 1024)), dev((1024, 1024))])
    with pytest.raises(ValueError, match="holds float"):
        p.check([scal, dev((1024, 1024), np.float64), dev((1024, 1024)), dev((1024, 1024))])
    with pytest.raises(ValueError, match="device memory"):
        p.check([scal, runtime.Buffer.from_numpy(np.zeros((1024, 1024), np.float32)), dev((1024, 1024)), dev((1024, 1024))])
