"""GPU parity tests: the reference's own GPU test programs (tests/test_167.cpp ... of the
reference tree), compiled by the HIP back-end and compared with the nested-loop references
their wrappers use.  Inputs are small integers, as in the reference, so fp32 results are
exact and the comparison is bit-for-bit."""
import numpy as np
import pytest

from oracle import reference_loops as ref
from tiramisu_amd import runtime

pytestmark = pytest.mark.gpu


def _ints(rng, shape):
    return (rng.randint(0, 10, shape) - 5).astype(np.float32)


def test_167_gemm_gpu_tile(programs_dir):
    prog = runtime.load(programs_dir, "test_167")
    rng = np.random.RandomState(167)
    A, B, C = _ints(rng, (128, 128)), _ints(rng, (128, 128)), _ints(rng, (128, 128))
    expected = ref.gemm_accumulate(A, B, C)
    prog(A, B, C)
    assert np.array_equal(C, expected)
