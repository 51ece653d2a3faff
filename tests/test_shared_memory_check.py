"""The race check of shared memory (back-end option hip_check_shared_memory; the reference leaves barriers to the
program, tiramisu_codegen_cuda.cpp:1240-1242, and checks nothing).  tests/programs/shared_memory_check.cpp stages
64 elements per workgroup in an LDS buffer declared by hand and reads what another thread wrote: with the barriers
the check accepts the programs and the kernels give numpy's result on the GPU; with a barrier left out the generator
must stop (or, in `warn` mode, print the finding and go on).  Programs whose barriers cache_shared() places, and
from which the emitter drops the redundant ones, must pass the check as well."""
import os
import subprocess

import numpy as np
import pytest

from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_generator(gen, tmp_path, *args, env=None):
    os.makedirs(os.path.join(str(tmp_path), "build"), exist_ok=True)
    full = dict(os.environ)
    full.update(env or {})
    return subprocess.run([gen] + list(args), cwd=str(tmp_path), env=full, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)


def test_synced_programs_pass_the_check(programs_dir, tmp_path):
    gen = os.path.join(programs_dir, "build", "gen_shared_memory_check")
    r = run_generator(gen, tmp_path, "--backend-option", "hip_check_shared_memory=1")
    assert r.returncode == 0, r.stdout
    assert "LDS race check" not in r.stdout


@pytest.mark.parametrize("variant, first, second", [
    ("unsynced", "stage writes tile[c3]", "out reads tile[((-c3) + 63)]"),
    # the hazard across iterations of the serial loop in the kernel: the read of one round, the write of the next
    ("one_sync", "sum reads tile[((-c3) + 63)]", "stage writes tile[c3]"),
])
def test_missing_barrier_stops_code_generation(programs_dir, tmp_path, variant, first, second):
    gen = os.path.join(programs_dir, "build", "gen_shared_memory_check")
    r = run_generator(gen, tmp_path, "--backend-option", "hip_check_shared_memory=1", variant)
    assert r.returncode != 0
    assert 'LDS race check: no sync between "%s" and "%s"' % (first, second) in r.stdout, r.stdout
    assert "element 0 is touched by thread" in r.stdout
    assert "shared-memory accesses of different threads are not separated by a sync" in r.stdout
    # warn: same finding, code generation goes on; without the option nothing is looked at
    r = run_generator(gen, tmp_path, "--backend-option", "hip_check_shared_memory=warn", variant)
    assert r.returncode == 0 and "LDS race check: no sync between" in r.stdout
    r = run_generator(gen, tmp_path, variant)
    assert r.returncode == 0 and "LDS race check" not in r.stdout


def test_cache_shared_programs_pass_the_check(programs_dir, tmp_path):
    """tests/programs/gemm_cache_shared.cpp kept as scheduled: cooperative copies into two LDS tiles in a serial loop,
    the barriers of cache_shared() with the redundant ones dropped by the emitter."""
    gen = os.path.join(programs_dir, "build", "gen_gemm_cache_shared")
    r = run_generator(gen, tmp_path, env={"TIRAMISU_HIP_CHECK_SHARED_MEMORY": "1"})
    assert r.returncode == 0, r.stdout
    assert "LDS race check" not in r.stdout
    text = open(os.path.join(str(tmp_path), "build", "gemm_u8_shared.o.hip")).read()
    assert "__shared__" in text and "__syncthreads" in text


@pytest.mark.parametrize("stem", ["sgemm_generator1", "sgemm_generator2", "sgemm_generator3"])
def test_reference_sgemm_generators_pass_the_check(tmp_path, stem):
    """The reference's benchmarks/linear_algebra/blas/level3/sgemm/gpu/generator{1,2,3}.cpp kept as scheduled
    (generator1 double-buffers its hand-declared LDS tiles, generator3 uses cache_shared): every access is
    analysed and none is reported."""
    gen = os.path.join(ROOT, "tests", "reference_programs", "build", stem, "gen")
    if not os.path.exists(gen):
        pytest.skip("the reference's generators are built only where its sources are")
    r = run_generator(gen, tmp_path, env={"TIRAMISU_HIP_CHECK_SHARED_MEMORY": "1", "TIRAMISU_NO_MFMA": "1"})
    assert r.returncode == 0, r.stdout
    assert "LDS race check" not in r.stdout
    text = open(os.path.join(str(tmp_path), "fct.o.hip")).read()
    assert "__shared__" in text and "__syncthreads" in text


STUBS = {"HIPCC_PATH": "/bin/true", "TIRAMISU_HOST_CXX": "/bin/true"}      # the check runs before any code is emitted


@pytest.mark.parametrize("gen", ["gen_convolutiongpu_tiramisu", "gen_heat2dgpu_tiramisu", "gen_tutorial_04gpu2"])
def test_reference_programs_with_run_time_sizes_are_analysed_and_pass(tmp_path, gen):
    """benchmarks/halide/convolutiongpu_tiramisu.cpp (an 18 x 18 LDS tile filled by four guarded copies),
    heat2dgpu_tiramisu.cpp and tutorial_04gpu2: image sizes known only at run time, so the thread loops' bounds are
    min(15, N - 16 block - 1) and the halo copies' guards mix thread and size terms; the check takes the constant
    side of such bounds and the decidable side of such guards, analyses every access and finds nothing."""
    path = os.path.join(ROOT, "tests", "reference_programs", "build", gen)
    if not os.path.exists(path):
        pytest.skip("the reference's generators are built only where its sources are")
    r = run_generator(path, tmp_path, env=dict(STUBS, TIRAMISU_HIP_CHECK_SHARED_MEMORY="1"))
    assert r.returncode == 0, r.stdout[-2000:]
    assert "LDS race check" not in r.stdout


def test_the_reference_hand_staged_lstm_has_races(tmp_path):
    """benchmarks/DNN/blocks/LSTM/gpu/generator.cpp:212-236 orders, inside the loop over 16-wide slices, the product
    that reads the LDS tiles, one sync, the stores of the next slice into the tiles -- and then the next round's
    product with nothing in between (and for the second product: stores, sync, product, next round's stores).  The
    check names all four: a write of one round against the reads of the next on both tiles of the first product,
    reads against the next round's writes on both tiles of the second."""
    path = os.path.join(ROOT, "tests", "reference_programs", "build", "lstm_gpu", "gen")
    if not os.path.exists(path):
        pytest.skip("the reference's generators are built only where its sources are")
    r = run_generator(path, tmp_path, env=dict(STUBS, TIRAMISU_HIP_CHECK_SHARED_MEMORY="warn"))
    assert r.returncode == 0, r.stdout[-2000:]
    found = [l for l in r.stdout.split("\n") if l.startswith("LDS race check: no sync between")]
    assert len(found) == 4, r.stdout[-3000:]
    for tile, first in (("b_m1_R_shr", "writes"), ("b_m1_h_shr", "writes"), ("b_m2_W_shr", "reads"), ("b_m2_h_shr", "reads")):
        assert any((first + " " + tile) in l.split('" and "')[0] and tile in l.split('" and "')[1] for l in found), tile
    # with "1" the same findings stop code generation
    r = run_generator(path, tmp_path, env=dict(STUBS, TIRAMISU_HIP_CHECK_SHARED_MEMORY="1"))
    assert r.returncode != 0 and "not separated by a sync" in r.stdout


@pytest.mark.gpu
def test_gpu_kernels_with_hand_declared_lds_match_numpy(programs_dir):
    from gpu_util import DeviceArray
    rng = np.random.RandomState(5)
    src = (rng.randint(0, 100, (64, 64)) - 50).astype(np.float32)
    for name, expected in (("reverse_in_blocks", src[:, ::-1]),
                           ("sums_over_rounds", 5 * src[:, ::-1] + 10)):
        prog = runtime.load(programs_dir, name)
        dev = [DeviceArray(src), DeviceArray(np.full((64, 64), -7.0, np.float32))]
        print("running", name, flush=True)
        prog(*[d.buffer() for d in dev])
        got = dev[-1].download()
        for d in dev:
            d.free()
        assert np.array_equal(got, expected.astype(np.float32)), name
