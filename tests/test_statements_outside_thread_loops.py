"""Statements of a kernel that no thread loop encloses (tests/programs/statements_outside_thread_loops.cpp): the
program means them to run once per iteration of the block loops around them; the reference's CUDA printer emits
them as code of every thread (tiramisu_codegen_cuda.cpp: a thread loop becomes an index and a guard, what lies
outside is left alone), which is a race for an accumulation.  The HIP back-end runs them on the workgroup's first
thread between barriers; back-end option hip_every_thread_runs_all gives the other form."""
import os
import subprocess

import numpy as np
import pytest

from tiramisu_amd import runtime

NAME = "weights_outside_thread_loops"


def test_kernel_runs_them_on_the_first_thread_between_barriers(programs_dir):
    text = open(os.path.join(programs_dir, "build", NAME + ".o.hip")).read()
    assert "statements outside the thread loops run on the workgroup's first thread between barriers" in text
    kernel = text[text.index('extern "C" __global__'):]
    guard = kernel.index("if (threadIdx.x == 0) {")
    thread_loop = kernel.index("(int32_t)threadIdx.x + 0")
    barriers = [i for i in range(len(kernel)) if kernel.startswith("__syncthreads();", i)]
    assert len(barriers) == 2 and barriers[0] < guard < barriers[1] < thread_loop
    # the accumulation is inside the guarded region
    assert guard < kernel.index("_weight_init_b1[c1] = (_weight_init_b1[c1] + ") < barriers[1]


def test_the_other_form_is_an_option(programs_dir, tmp_path):
    os.makedirs(os.path.join(str(tmp_path), "build"))
    env = dict(os.environ, HIPCC_PATH="/bin/true", TIRAMISU_HOST_CXX="/bin/true")
    r = subprocess.run([os.path.join(programs_dir, "build", "gen_statements_outside_thread_loops"), "--backend-option", "hip_every_thread_runs_all=1"],
                       cwd=str(tmp_path), env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    text = open(os.path.join(str(tmp_path), "build", NAME + ".o.hip")).read()
    assert "__syncthreads" not in text and "once per workgroup" not in text


def test_loop_level_tagged_block_by_some_statements_and_thread_by_others_is_a_block_dimension(programs_dir):
    """weights_under_conflicting_tags: the weights tag (b, c) as (block, thread), the output tags (b, c, u, t) as
    (block, block, thread, thread), and they are fused at c -- as the reference's dibaryon correlators fuse their
    two-level and four-level statements.  c is a block dimension; the weights run once per workgroup."""
    text = open(os.path.join(programs_dir, "build", "weights_under_conflicting_tags.o.hip")).read()
    assert "a loop tagged as a block dimension by some statements and as a thread dimension by others is a block dimension" in text
    kernel = text[text.index('extern "C" __global__'):]
    assert "const int32_t c3 = (int32_t)_tile.x" in kernel or "const int32_t c3 = (int32_t)blockIdx.x" in kernel
    guard = kernel.index("if (threadIdx.x == 0 && threadIdx.y == 0) {")
    assert guard < kernel.index("(int32_t)threadIdx.y + 0")
    host = open(os.path.join(programs_dir, "build", "weights_under_conflicting_tags.o.host.cpp")).read()
    assert "_grid[3] = {(uint32_t)(5), (uint32_t)(6), (uint32_t)(1)}" in host and "_block[3] = {(uint32_t)(16), (uint32_t)(4), (uint32_t)(1)}" in host


@pytest.mark.gpu
def test_gpu_conflicting_tags_match_the_sequential_meaning(programs_dir):
    from gpu_util import DeviceArray
    shape = (6, 5, 4, 16)
    rng = np.random.RandomState(22)
    src = (rng.randint(0, 50, shape) - 25).astype(np.float32)
    dev = [DeviceArray(src), DeviceArray(np.full(shape[:2], -7.0, np.float32)), DeviceArray(np.full(shape, -7.0, np.float32))]
    print("running weights_under_conflicting_tags", flush=True)
    runtime.load(programs_dir, "weights_under_conflicting_tags")(*[d.buffer() for d in dev])
    weight, out = dev[1].download(), dev[2].download()
    for d in dev:
        d.free()
    assert np.array_equal(weight, np.full(shape[:2], 15.0, np.float32))
    assert np.array_equal(out, src + 15.0)


@pytest.mark.gpu
def test_gpu_matches_the_sequential_meaning(programs_dir):
    from gpu_util import DeviceArray
    NB, T = 48, 64
    rng = np.random.RandomState(21)
    src = (rng.randint(0, 50, (NB, T)) - 25).astype(np.float32)
    dev = [DeviceArray(src), DeviceArray(np.full((NB,), -7.0, np.float32)), DeviceArray(np.full((NB, T), -7.0, np.float32))]
    print("running", NAME, flush=True)
    runtime.load(programs_dir, NAME)(*[d.buffer() for d in dev])
    weight, out = dev[1].download(), dev[2].download()
    for d in dev:
        d.free()
    assert np.array_equal(weight, np.full((NB,), 15.0, np.float32))
    assert np.array_equal(out, src + 15.0)
