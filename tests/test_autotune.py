"""Evaluation by execution.  tiramisu_amd.autotune: option combinations, argument construction from the back-end's
description of a function, the argument check in runtime.Program, and two candidates of one program -- option
sets handed to the generator as --backend-option arguments, nothing through the environment -- generated ahead of
time (no GPU needed: the generator calls hipcc), then timed on the GPU, which must give equal results and a
positive time for each.  The C++ class tiramisu::auto_scheduler::evaluate_by_execution (the reference's
include/tiramisu/auto_scheduler/evaluator.h:34-80) is driven through the compiled tuner
tiramisu_amd/tuning/square_tiles.cpp: without a GPU with a stand-in wrapper command (candidates are generated,
compiled, linked, their options recorded in the manifest), on the GPU with the real wrapper, whose kept outputs
must be alpha * A x B + beta * C."""
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


# ---------------------------------------------------------------- evaluation by execution

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EVAL_DIR = os.path.join(ROOT, "tests", "programs", "build", "evaluate_by_execution")
CANDIDATES = [{"mfma_bk": "16"}, {"mfma_bk": "32"}]      # back-end options (function::set_backend_option)


def evaluator():
    return autotune.evaluate_by_execution(os.path.join(ROOT, "tests", "programs", "gemm_gpu_tile.cpp"), "gemm_gpu_tile", EVAL_DIR, repeat=10)


def test_candidates_are_prepared_without_a_gpu():
    ev = evaluator()
    for c in CANDIDATES:
        lib = ev.prepare(c)
        assert os.path.exists(lib)
        slices = "x%s," % c["mfma_bk"]
        assert any(slices in k["how"] for k in runtime.manifest_of(lib, "gemm_gpu_tile")["kernels"])   # the option reached the emitter
        assert ev.options_used(c) == c and "TIRAMISU_MFMA_BK" not in os.environ


@pytest.mark.gpu
def test_evaluate_by_execution_times_candidates_on_the_gpu():
    ev = evaluator()
    outputs, times = [], []
    for c in CANDIDATES:
        if not os.path.exists(ev.library(c)):
            pytest.skip("candidates were not prepared (run the CPU test suite or __graft_entry__.build() first)")
        print("evaluating", c, flush=True)
        samples = ev.get_measurements(c, repeat=10)
        assert len(samples) == 10 and all(t > 0 for t in samples)
        times.append(ev.evaluate(c))
        outputs.append(ev.last_outputs)
        assert ev.last_kernels[0].startswith("mfma-contraction")
    assert all(t > 0 for t in times)
    assert all(np.array_equal(a, b) for a, b in zip(outputs[0], outputs[1]))
    # the result is the program's: C += A x B on the harness's seeded integer inputs
    m = runtime.manifest_of(ev.library(CANDIDATES[0]), "gemm_gpu_tile")
    A, B, C = autotune.make_arguments(m, ev.seed)
    assert np.array_equal(outputs[0][0], C + A @ B)


# ---------------------------------------------------------------- the C++ evaluator, through a compiled tuner

TUNER_DIR = os.path.join(ROOT, "tests", "programs", "build", "square_tiles")


def test_cpp_evaluator_generates_compiles_and_links_every_candidate():
    """No GPU: the wrapper command is a stand-in that prints three times.  The tuner must have generated the
    program once per candidate on one tiramisu::function, and the last manifest records the candidate's option."""
    import json
    import shutil
    shutil.rmtree(TUNER_DIR, ignore_errors=True)
    lines = autotune.run_tuner("square_tiles", TUNER_DIR, "--wrapper", "echo 1.5 2.5 3.5 #", 256)
    assert len(lines) == 1
    r = lines[0]
    assert r["size"] == 256 and r["model_tile"] in (64, 128, 256)
    assert set(r["ms"]) == {"default", "64", "128", "256"} and all(v == 2.5 for v in r["ms"].values())   # medians of the stand-in
    m = json.load(open(os.path.join(TUNER_DIR, "sgemm_tiles_256.o.json")))
    assert m["options"] == [{"name": "mfma_tile", "value": "256", "from": "program"}]
    assert "tile 256x256x16" in m["kernels"][0]["how"]
    assert os.path.exists(os.path.join(TUNER_DIR, "sgemm_tiles_256.o.so"))


@pytest.mark.gpu
def test_cpp_evaluator_times_candidates_and_reproduces_the_product(tmp_path):
    outputs = str(tmp_path / "outputs.npz")
    wrapper = "python3 -m tiramisu_amd.autotune --time --repeat 5 --outputs " + outputs
    lines = autotune.run_tuner("square_tiles", str(tmp_path), "--wrapper", wrapper, 256)
    r = lines[0]
    print(r, flush=True)
    assert all(0 < v < 1e3 for v in r["ms"].values())
    assert str(r["fastest_tile"]) in r["ms"]
    got = np.load(outputs)
    scal, A, B, C0 = autotune.make_arguments(json.load(open(str(tmp_path / "sgemm_tiles_256.o.json"))), 1)   # the wrapper's seeded inputs
    expected = scal[0] * (A.host.astype(np.float64) @ B.host.astype(np.float64)) + scal[1] * C0.host
    assert np.array_equal(got["b_C"], expected.astype(np.float32))
    for a in (A, B, C0):
        a.free()
