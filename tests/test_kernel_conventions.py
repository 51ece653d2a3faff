"""Conventions of the generated kernel text that the reference's CUDA back-end fixes and generated
host code or tools may rely on, pinned by the sample of generated CUDA the reference tree holds
(benchmarks/DNN/blocks/MULTI_GPU_4LSTM_MaxPool_4LSTM/multi_gpu_deepspeech_kernels.cu:12-34, :326-356):
kernels are called _kernel_<n> with n counting up through the process (tiramisu_codegen_cuda.cpp:1320),
parameters are the scalars, sorted by name, then the buffers, sorted by name (:1324-1331), loop
iterators are c1, c3, ... and the block / thread index is added to the loop's lower bound."""
import glob
import os
import re

SIGNATURE = re.compile(r'^extern "C" __global__ void __launch_bounds__\((\d+)(?:, \d+)?\)\s*(?:__attribute__\(\([^)]*\)\)\s*)?(_kernel_(\d+))\(([^)]*)\)', re.M)


def kernels_of(path):
    return [(m.group(2), int(m.group(3)), [p.strip() for p in m.group(4).split(",") if p.strip()], int(m.group(1)))
            for m in SIGNATURE.finditer(open(path).read())]


def generic_sources(programs_dir):
    files = sorted(glob.glob(os.path.join(programs_dir, "build", "*.o.hip")))
    assert files, "run __graft_entry__.build() first"
    return files


def test_scalars_then_buffers_each_sorted_by_name(programs_dir):
    seen = 0
    for path in generic_sources(programs_dir):
        for name, number, params, threads in kernels_of(path):
            assert 1 <= threads <= 1024
            scalars = [p for p in params if "*" not in p]
            buffers = [p for p in params if "*" in p]
            assert params == scalars + buffers, (path, name)
            names = lambda ps: [p.split()[-1].lstrip("*") for p in ps]
            assert names(scalars) == sorted(names(scalars)), (path, name)
            assert names(buffers) == sorted(names(buffers)), (path, name)
            assert all(p.startswith("const ") for p in scalars) and all("__restrict__" in p for p in buffers)
            seen += 1
    assert seen >= 20


def test_kernels_are_numbered_through_the_generating_process(programs_dir):
    # one generator program emits several functions: the counter does not restart between them
    numbers = []
    for name in ("sgemm_shared_regs", "sgemm_shared_regs_generic", "gemm_u8_shared"):   # tests/programs/gemm_cache_shared.cpp
        numbers += [n for _, n, _, _ in kernels_of(os.path.join(programs_dir, "build", name + ".o.hip"))]
    assert sorted(numbers) == list(range(len(numbers)))


def test_iterators_and_index_expressions(programs_dir):
    # block / thread loops become the hardware index plus the loop's lower bound, named like isl's iterators
    # (a kernel with a one-dimensional grid: two-dimensional ones may deal their points out again)
    plain = open(os.path.join(programs_dir, "build", "row_sums_quarter_wave.o.hip")).read()
    assert re.search(r"const int32_t c\d+ = \(int32_t\)blockIdx\.[xyz] \+ 0;", plain)
    assert re.search(r"const int32_t c\d+ = \(int32_t\)threadIdx\.[xyz] \+ 0;", plain)
    text = open(os.path.join(programs_dir, "build", "parallel_host_loop_serial.o.hip")).read()
    # a host loop iterator reaches the kernel as a scalar parameter of the same name
    assert re.search(r"_kernel_\d+\(const int32_t c1, float \*__restrict__ b_base, float \*__restrict__ b_s1\)", text)
