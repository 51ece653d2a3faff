"""Writes the small regression fixtures of this directory from the oracle (oracle/reference_loops.py).

The reference tree holds no data files for the GPU code-generation path: its tests compute their
expected values with nested loops inside the wrapper programs (tests/wrapper_test_162.cpp:28-35,
wrapper_test_167.cpp:21-28, wrapper_test_168.cpp:8-19, wrapper_test_197.cpp:8-41), and those loops
are what the oracle restates.  The fixtures here therefore pin the oracle against *itself over
time*: inputs (seeded) and the outputs the pinned oracle gave when they were written, so that a
later change of the oracle, of the CPU-generated code or of a kernel that alters a result shows up
as a diff against committed bytes.  Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import reference_loops as ref  # noqa: E402


def ints(rng, shape):
    return (rng.randint(0, 10, shape) - 5).astype(np.float32)


def main():
    rng = np.random.RandomState(20240607)
    # sgemm 33x17x9, alpha 2 beta -1 (integer data: exact)
    A, B, C = ints(rng, (33, 9)), ints(rng, (9, 17)), ints(rng, (33, 17))
    np.savez(os.path.join(HERE, "sgemm_33x17x9.npz"), A=A, B=B, C=C, alpha=np.float32(2), beta=np.float32(-1),
             out=ref.sgemm(A, B, C, 2.0, -1.0))
    # heat2d 20x20, 2 steps
    g = np.zeros((20, 20), np.float32)
    g[1:-1, 1:-1] = rng.uniform(0, 1, (18, 18)).astype(np.float32)
    np.savez(os.path.join(HERE, "heat2d_20x2.npz"), grid=g, planes=ref.heat2d(g, 2))
    # conv2d 1x3x5x12 (N, CI, CO, H), padded input
    xp = np.zeros((1, 3, 14, 14), np.float32)
    xp[:, :, 1:-1, 1:-1] = ints(rng, (1, 3, 12, 12))
    w, b = ints(rng, (5, 3, 3, 3)), ints(rng, (5,))
    np.savez(os.path.join(HERE, "conv2d_1x3x5x12.npz"), x=xp, w=w, b=b, out=ref.conv2d_bias_relu(xp, w, b))
    # lstm 1 layer, batch 4, hidden 16, 3 steps
    wl = rng.uniform(-0.08, 0.08, (1, 2, 64, 16)).astype(np.float32)
    bl = rng.uniform(-0.08, 0.08, (1, 64)).astype(np.float32)
    xl = rng.uniform(-1, 1, (3, 4, 16)).astype(np.float32)
    np.savez(os.path.join(HERE, "lstm_1x4x16x3.npz"), w=wl, b=bl, x=xl, y=ref.lstm(wl, bl, xl))
    # bilinear resampling 90x132
    src = rng.randint(0, 256, (90, 132)).astype(np.uint8)
    np.savez(os.path.join(HERE, "resample_bilinear_90x132.npz"), src=src, out=ref.resample_bilinear(src))


if __name__ == "__main__":
    main()
