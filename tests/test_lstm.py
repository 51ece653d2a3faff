"""Stacked LSTM (benchmark configuration 5): oracle pins, CPU-generated code vs the oracle, and the GPU
program (per cell one MFMA kernel: both gate products, bias and the element-wise cell update on the
finished tile; the independent cells of a diagonal of (layer, time step) in one launch) vs both.

Tolerance: max |gpu - ref| <= 1e-4 * max |ref| on the output sequence y (fp32; the MFMA kernel
sums in a different order and the device's expf/tanhf differ from libm in the last ulps)."""
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from oracle import reference_loops as ref
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")
SMALL = [(2, 8, 32, 5), (1, 4, 16, 3), (3, 20, 64, 4), (2, 64, 256, 6)]
RTOL = 1e-4


def name_of(s):
    return "lstm_%dx%dx%dx%d" % s


def cpu_program(s):
    return runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name_of(s)), name_of(s), needs_gpu_runtime=False)


def make_inputs(s, seed):
    L, B, H, S = s
    rng = np.random.RandomState(seed)
    w = rng.uniform(-0.08, 0.08, (L, 2, 4 * H, H)).astype(np.float32)
    b = rng.uniform(-0.08, 0.08, (L, 4 * H)).astype(np.float32)
    x = rng.uniform(-1.0, 1.0, (S, B, H)).astype(np.float32)
    return w, b, x


# ---------------------------------------------------------------- oracle pins

def test_oracle_against_torch_lstm():
    # textbook LSTM with gate order i, f, g, o and a single bias: torch.nn.LSTM with b_hh = 0
    import torch
    s = (2, 3, 8, 6)
    w, b, x = make_inputs(s, 11)
    L, B, H, S = s
    net = torch.nn.LSTM(H, H, num_layers=L)
    with torch.no_grad():
        for l in range(L):
            getattr(net, "weight_ih_l%d" % l).copy_(torch.from_numpy(w[l, 0]))
            getattr(net, "weight_hh_l%d" % l).copy_(torch.from_numpy(w[l, 1]))
            getattr(net, "bias_ih_l%d" % l).copy_(torch.from_numpy(b[l]))
            getattr(net, "bias_hh_l%d" % l).zero_()
        y, _ = net(torch.from_numpy(x))
    assert np.allclose(ref.lstm(w, b, x), y.numpy(), rtol=1e-5, atol=1e-6)


def test_oracle_zero_weights_closed_form():
    # with W = R = 0 every sample follows c_t = s(b_i) tanh(b_z) + s(b_f) c_{t-1}, h_t = tanh(c_t) s(b_o)
    s = (1, 2, 4, 5)
    w, b, x = make_inputs(s, 12)
    w[:] = 0
    y = ref.lstm(w, b, x)
    sig = lambda v: 1.0 / (1.0 + np.exp(-v.astype(np.float64)))
    H = 4
    c = np.zeros(H)
    for t in range(5):
        c = sig(b[0, 0:H]) * np.tanh(b[0, 2 * H:3 * H].astype(np.float64)) + sig(b[0, H:2 * H]) * c
        h = np.tanh(c) * sig(b[0, 3 * H:4 * H])
        assert np.allclose(y[t], np.broadcast_to(h, (2, H)), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("s", SMALL)
def test_cpu_generated_code_matches_oracle(s):
    w, b, x = make_inputs(s, sum(s))
    y = np.zeros((s[3], s[1], s[2]), np.float32)
    cpu_program(s)(w, b, x, y)
    expected = ref.lstm(w, b, x)
    assert np.max(np.abs(y - expected)) <= 1e-5 * np.max(np.abs(expected))


# ---------------------------------------------------------------- GPU parity

def run_gpu(s, w, b, x):
    from gpu_util import DeviceArray
    y = np.zeros((s[3], s[1], s[2]), np.float32)
    d = [DeviceArray(a) for a in (w, b, x, y)]
    runtime.load(PROGRAMS, name_of(s))(*[q.buffer() for q in d])
    out = d[3].download()
    for q in d:
        q.free()
    return out


@pytest.mark.parametrize("s", SMALL + [(4, 64, 512, 100)])
def test_cell_is_one_fused_kernel(s):
    """The gate contraction takes the element-wise nest that follows it into its kernel (the four gate
    columns of a hidden unit in one workgroup), the gate buffer and the four activation temporaries stay
    in registers, and -- with more than one layer -- the cells of a diagonal share a launch."""
    import json
    kernels = json.load(open(os.path.join(PROGRAMS, "build", name_of(s) + ".o.json")))["kernels"]
    fused = [k["how"] for k in kernels if k["how"].startswith("mfma-contraction")]
    assert len(fused) == 1 and len(kernels) == 5          # h_init, c_init, copy of x, the cell, y
    assert "2 product term(s), fused initialisation, 9 point-wise statement(s) of the following nest fused" in fused[0]
    assert "4 column group(s) per unit, 5 temporaries kept in registers" in fused[0]
    assert ("gridDim.z" in fused[0]) == (s[0] > 1)


@pytest.mark.gpu
@pytest.mark.parametrize("s", SMALL)
def test_gpu_matches_cpu_generated_code(s):
    w, b, x = make_inputs(s, 7 + sum(s))
    y_cpu = np.zeros((s[3], s[1], s[2]), np.float32)
    cpu_program(s)(w, b, x, y_cpu)
    y = run_gpu(s, w, b, x)
    from gpu_util import assert_fp32_parity
    assert_fp32_parity(y, y_cpu, "lstm %s vs CPU-generated code" % (s,), RTOL)
    assert_fp32_parity(y, ref.lstm(w, b, x), "lstm %s vs numpy oracle" % (s,), RTOL)


@pytest.mark.gpu
def test_gpu_full_size_matches_oracle():
    s = (4, 64, 512, 100)
    w, b, x = make_inputs(s, 512)
    y = run_gpu(s, w, b, x)
    expected = ref.lstm(w, b, x)
    from gpu_util import assert_fp32_parity
    assert_fp32_parity(y, expected, "lstm full size vs numpy oracle", RTOL)
    # zero weights: every time step of every sample equals the closed-form recurrence
    w0 = np.zeros_like(w)
    y0 = run_gpu(s, w0, b, x)
    assert np.max(np.abs(y0 - ref.lstm(w0, b, x))) <= 1e-6
    assert np.all(np.abs(y0 - y0[:, :1, :]) == 0)   # no dependence on the sample
