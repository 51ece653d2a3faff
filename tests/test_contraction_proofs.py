"""What the HIP back-end proves before a scheduled GEMM nest becomes its MFMA kernel
(tests/programs/contraction_proofs.cpp): LDS tiles installed with cache_shared must hold exactly
what the nest reads through them, and no two results of a thread may share an element of its
register tile; a fused epilogue may read the accumulator only at its own element.  The flawed
schedules stay as scheduled; they are generated, not run."""
import os
import re

import numpy as np
import pytest

from oracle import reference_loops as ref
from tiramisu_amd import runtime


def kernel_kind(programs_dir, name):
    text = open(os.path.join(programs_dir, "build", name + ".o.hip")).read()
    return re.search(r"^// _kernel_\d+: ([a-z-]+)", text, re.M).group(1)


@pytest.mark.parametrize("name,kind", [
    ("proofs_sound", "mfma-contraction"),
    ("proofs_short_tile", "generic"),
    ("proofs_shifted_tile", "generic"),
    ("proofs_unaligned_tile", "generic"),
    ("proofs_shared_register", "generic"),
    ("proofs_epilogue_other_element", "generic"),
])
def test_kernel_chosen(programs_dir, name, kind):
    assert kernel_kind(programs_dir, name) == kind


@pytest.mark.gpu
def test_sound_schedule_computes_the_gemm(programs_dir):
    rng = np.random.RandomState(26)
    M, N, K = 256, 256, 128
    A = rng.randint(-3, 4, (M, K)).astype(np.float32)
    B = rng.randint(-3, 4, (K, N)).astype(np.float32)
    C = rng.randint(-3, 4, (M, N)).astype(np.float32)
    expected = ref.sgemm(A, B, C, 1.0, 1.0)
    from gpu_util import DeviceArray
    dA, dB, dC = DeviceArray(A), DeviceArray(B), DeviceArray(C)
    runtime.load(programs_dir, "proofs_sound")(dA.buffer(), dB.buffer(), dC.buffer())
    assert np.array_equal(dC.download(), expected)
