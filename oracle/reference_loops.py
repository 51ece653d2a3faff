"""numpy restatements of the reference's in-tree nested-loop references (test infrastructure).

Every function cites the reference lines it restates.  Pins (what fixes each function's
behaviour independently of this file) are exercised in tests/test_oracle.py.
"""
import numpy as np


def gemm_accumulate(A, B, C):
    """C + A.B, row-major.  Reference: tests/wrapper_test_167.cpp:21-28 (Halide::Buffer indices
    are flipped there: C_ref(i, j) += A(k, j) * B(i, k) is C[j][i] += A[j][k] * B[k][i]).
    Accumulation order is k ascending from the initial C, in fp32, like the reference loop."""
    out = C.astype(np.float32).copy()
    K = A.shape[1]
    for k in range(K):
        out += np.outer(A[:, k], B[k, :]).astype(np.float32)
    return out


def sgemm(A, B, C, alpha, beta):
    """alpha*A.B + beta*C.  Reference: tests/wrapper_test_162.cpp:28-35 and
    benchmarks/linear_algebra/blas/level3/sgemm/cpu/sgemm_wrapper.cpp:166-169."""
    acc = np.zeros((A.shape[0], B.shape[1]), dtype=np.float32)
    for k in range(A.shape[1]):
        acc += np.outer(A[:, k], B[k, :]).astype(np.float32)
    return (np.float32(alpha) * acc + np.float32(beta) * C.astype(np.float32)).astype(np.float32)


def transpose(A):
    """Reference: tests/wrapper_test_168.cpp:8-19."""
    return np.ascontiguousarray(A.T)
