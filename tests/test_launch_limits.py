"""The limits of a workgroup (tests/programs/launch_limits.cpp): 1024 threads and 160 KiB of shared memory are checked
when the code is generated -- the device compiler accepts more and the launch would fail (the reference leaves both to
nvcc and to the launch, tiramisu_codegen_cuda.cpp:1356-1371) -- and a kernel exactly at both limits runs."""
import os
import subprocess

import numpy as np
import pytest

from tiramisu_amd import runtime

STUBS = {"HIPCC_PATH": "/bin/true", "TIRAMISU_HOST_CXX": "/bin/true"}


def generate(programs_dir, tmp_path, *args):
    os.makedirs(os.path.join(str(tmp_path), "build"), exist_ok=True)
    return subprocess.run([os.path.join(programs_dir, "build", "gen_launch_limits")] + list(args), cwd=str(tmp_path), env=dict(os.environ, **STUBS),
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)


def test_the_kernel_at_the_limits_is_generated(programs_dir, tmp_path):
    r = generate(programs_dir, tmp_path)
    assert r.returncode == 0, r.stdout
    text = open(os.path.join(programs_dir, "build", "at_the_limits.o.hip")).read()
    assert "__launch_bounds__(1024)" in text and "__shared__ float tile[40960];" in text


def test_too_many_threads_stop_code_generation(programs_dir, tmp_path):
    r = generate(programs_dir, tmp_path, "threads")
    assert r.returncode != 0
    assert "kernel _kernel_1 of too_many_threads: a workgroup of 64 x 64 x 1 = 4096 threads; the limit is 1024" in r.stdout, r.stdout


def test_too_much_shared_memory_stops_code_generation(programs_dir, tmp_path):
    r = generate(programs_dir, tmp_path, "lds")
    assert r.returncode != 0
    assert "of too_much_shared_memory: 163844 bytes of shared memory; a workgroup has 163840" in r.stdout, r.stdout


@pytest.mark.gpu
def test_the_kernel_at_the_limits_runs(programs_dir):
    from gpu_util import DeviceArray
    rng = np.random.RandomState(160)
    src = rng.randint(-50, 50, (6, 40, 32, 32)).astype(np.float32)
    # out is indexed (b, y, x, r): out(b, y, x, r) = in(b, 39 - r, 31 - y, 31 - x)
    expected = np.transpose(src[:, ::-1, ::-1, ::-1], (0, 2, 3, 1)).copy()
    dev = [DeviceArray(src), DeviceArray(np.full((6, 32, 32, 40), -7.0, np.float32))]
    print("at_the_limits", flush=True)
    runtime.load(programs_dir, "at_the_limits")(*[d.buffer() for d in dev])
    got = dev[1].download()
    for d in dev:
        d.free()
    assert np.array_equal(got, expected)
