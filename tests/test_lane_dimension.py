"""Which tagged thread loop runs along the lanes, how wide a workgroup is and which tile it takes
(tests/programs/lane_dimension.cpp): the kernel gives threadIdx.x to the loop along which the accesses have unit
stride and deals independent points out to workgroups one wavefront wide, unless a sum across threads ties the
mapping down.  The generated text is checked here without a GPU; results on the GPU against numpy and
against the CPU-generated code of the same programs, bit for bit (small integers)."""
import os
import re

import numpy as np
import pytest

from oracle import build as oracle_build
from tiramisu_amd import runtime


def kernel_source(programs_dir, name):
    return open(os.path.join(programs_dir, "build", name + ".o.hip")).read()


def on_gpu(programs_dir, name, *arrays):
    """Calls the generated function on device copies of `arrays` and returns the last one's contents."""
    from gpu_util import DeviceArray
    dev = [DeviceArray(a) for a in arrays]
    print("running", name, flush=True)
    runtime.load(programs_dir, name)(*[d.buffer() for d in dev])
    got = dev[-1].download()
    for d in dev:
        d.free()
    return got


def cpu_variant(programs_dir, name):
    return runtime.Program(oracle_build.cpu_program_library(programs_dir, name), name, needs_gpu_runtime=False)


def test_threadidx_x_follows_the_unit_stride(programs_dir):
    text = kernel_source(programs_dir, "lanes_follow_unit_stride")
    assert "threadIdx.x given to the thread loop along which the accesses have unit stride" in text
    # the points are dealt out again to workgroups one wavefront wide; the iterator that follows threadIdx.x is
    # the one added to the store index without a factor
    assert "points dealt out again to workgroups of 64 x 4 (the program's tiles: 16 x 16)" in text
    assert re.search(r"const uint32_t _g0 = blockIdx\.x \* 64u \+ threadIdx\.x;", text)
    assert re.search(r"const uint32_t _g1 = blockIdx\.y \* 4u \+ threadIdx\.y;", text)
    x_iterator = re.search(r"const int32_t (c\d+) = \(int32_t\)\(_g0 % 16u\)", text).group(1)
    y_iterator = re.search(r"const int32_t (c\d+) = \(int32_t\)\(_g1 % 16u\)", text).group(1)
    store = re.search(r"b_out\[(.*?)\] = ", text).group(1)
    assert re.search(r"\+ %s\) \* 150\)" % y_iterator, store) and re.search(r"\+ %s\)\)$" % x_iterator, store), store


def test_a_sum_across_threads_keeps_its_numbering(programs_dir):
    text = kernel_source(programs_dir, "column_sums_keep_lanes")
    assert "threadIdx.x given" not in text
    assert "sum(s) across the threads of a loop lowered to DPP wavefront reductions" in text


@pytest.mark.gpu
def test_gpu_lanes_follow_unit_stride(programs_dir):
    rng = np.random.RandomState(150)
    img = (rng.randint(0, 10, (70, 151)) - 5).astype(np.float32)
    out, out_cpu = np.full((70, 150), -1.0, np.float32), np.full((70, 150), -1.0, np.float32)
    cpu_variant(programs_dir, "lanes_follow_unit_stride")(img, out_cpu)
    out = on_gpu(programs_dir, "lanes_follow_unit_stride", img, out)
    assert np.array_equal(out, 2 * img[:, :150] + img[:, 1:])
    assert np.array_equal(out, out_cpu)


@pytest.mark.gpu
def test_gpu_column_sums(programs_dir):
    rng = np.random.RandomState(96)
    A = (rng.randint(0, 10, (192, 96)) - 5).astype(np.float32)
    s, s_cpu = np.full(96, -1.0, np.float32), np.full(96, -1.0, np.float32)
    cpu_variant(programs_dir, "column_sums_keep_lanes")(A, s_cpu)
    s = on_gpu(programs_dir, "column_sums_keep_lanes", A, s)
    assert np.array_equal(s, A.sum(axis=0))
    assert np.array_equal(s, s_cpu)


def test_workgroups_are_renumbered_where_tiles_share_data(programs_dir, product_programs_dir):
    # LDS staging (the cache_shared GEMM on the generic emitter): every XCD takes an eighth of the tiles;
    # a streaming kernel with wide tiles (the copy program; 600-byte-wide tiles here) keeps the hardware order
    shared = kernel_source(programs_dir, "sgemm_shared_regs_generic")
    assert "workgroups renumbered: an eighth of the tiles per XCD" in shared
    assert re.search(r"const int32_t c\d+ = \(int32_t\)_tile\.[xy] \+ 0;", shared) and "blockIdx.x + gridDim.x * blockIdx.y" in shared
    for text in (kernel_source(product_programs_dir, "copy_plane"), kernel_source(programs_dir, "lanes_follow_unit_stride")):
        assert "workgroups renumbered" not in text and "_tile" not in text


def test_the_mapping_passes_can_be_switched_off(programs_dir, tmp_path, monkeypatch):
    # the reference's own mapping: thread dimensions from the innermost tagged level outwards, the program's
    # tiles as workgroups, workgroups in hardware order
    from tiramisu_amd import build
    for knob in ("TIRAMISU_HIP_KEEP_THREAD_DIMENSIONS", "TIRAMISU_HIP_KEEP_TILES", "TIRAMISU_HIP_KEEP_BLOCK_ORDER"):
        monkeypatch.setenv(knob, "1")
    build.build_program(os.path.join(programs_dir, "lane_dimension.cpp"), directory=str(tmp_path))
    text = open(os.path.join(str(tmp_path), "build", "lanes_follow_unit_stride.o.hip")).read()
    assert "// _kernel_0: generic\n" in text
    # the innermost tagged loop (over y, the strided index) sits on threadIdx.x again
    x_iterator = re.search(r"const int32_t (c\d+) = \(int32_t\)threadIdx\.x \+ 0;", text).group(1)
    store = re.search(r"b_out\[(.*?)\] = ", text).group(1)
    assert re.search(r"\+ %s\) \* 150\)" % x_iterator, store), store
