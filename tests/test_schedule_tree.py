"""The AST from the schedule as a tree (back-end option ast_from_schedule_tree; tiramisu_amd/csrc/astgen.cpp).  The
reference hands isl one flat map from statement instances to time vectors (tiramisu_function.cpp: gen_isl_ast) and isl
derives the statements' order pairwise; the tree states it (a sequence per place among siblings, a band per loop).
With `check` a generator builds the AST both ways and reports whether the two lowered programs read the same; the
programs below -- tiled GPU nests, LDS staging, reductions across threads, parallel host loops, the skewed and
interchanged LSTM -- must, and a schedule that leaves a copy unordered against a loop nest must be left to the flat
form.  The device and host compilers are stubbed out: the comparison happens before any code is emitted."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(gen, tmp_path, mode, **extra):
    os.makedirs(os.path.join(str(tmp_path), "build"), exist_ok=True)
    env = dict(os.environ, TIRAMISU_AST_FROM_SCHEDULE_TREE=mode, HIPCC_PATH="/bin/true", TIRAMISU_HOST_CXX="/bin/true", **extra)
    r = subprocess.run([gen], cwd=str(tmp_path), env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:]
    return r.stdout


@pytest.mark.parametrize("where, stem, at_least", [
    ("tests/programs", "gemm_gpu_tile", 1), ("tests/programs", "gemm_cache_shared", 3), ("tests/programs", "thread_reductions", 3),
    ("tests/programs", "parallel_host_loop", 3), ("tests/programs", "shared_memory_check", 2), ("tests/programs", "host_loop_iterator_int64", 2),
    ("tiramisu_amd/programs", "lstm", 5), ("tiramisu_amd/programs", "conv2d", 4), ("tiramisu_amd/programs", "heat2d", 8),
])
def test_tree_and_map_give_the_same_program(tmp_path, where, stem, at_least):
    out = run(os.path.join(ROOT, where, "build", "gen_" + stem), tmp_path, "check")
    assert "another program text" not in out and "left to the flat form" not in out, out[-3000:]
    assert out.count("gives the same program both ways") >= at_least


def test_copy_left_unordered_against_a_loop_nest_is_left_to_the_flat_form(tmp_path):
    """The reference's benchmarks/DNN/blocks/LSTM/gpu/generator.cpp does not order the upload of x against the kernel
    that follows: the copy shares its place with the kernel's loops, and a band over both would scan it inside them."""
    gen = os.path.join(ROOT, "tests", "reference_programs", "build", "lstm_gpu", "gen")
    if not os.path.exists(gen):
        pytest.skip("the reference's generators are built only where its sources are")
    out = run(gen, tmp_path, "check")
    assert "is left to the flat form" in out and "another program text" not in out


def test_generated_code_is_the_same_file(tmp_path):
    """End to end with the real compilers switched off only for the device: the .hip file written with the option on
    is byte for byte the one written without it."""
    gen = os.path.join(ROOT, "tests", "programs", "build", "gen_gemm_cache_shared")
    texts = []
    for mode in ("0", "1"):
        d = tmp_path / mode
        d.mkdir()
        run(gen, d, mode)
        texts.append(open(os.path.join(str(d), "build", "sgemm_shared_regs_generic.o.hip")).read())
    assert texts[0] == texts[1] and "__global__" in texts[0]
