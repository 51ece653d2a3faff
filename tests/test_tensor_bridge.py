"""torch tensors as arguments of generated functions (tiramisu_amd/runtime.py: Buffer.from_tensor, Program.__call__;
the bridge that the reference's python_bindings leave to the caller -- its tutorials pass numpy arrays through
Halide buffers): no copy, host or GPU buffer by where the tensor lives, kernels in order with torch's work on the
tensor's stream."""
import os

import numpy as np
import pytest

from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")


def test_cpu_tensor_describes_a_host_buffer_without_a_copy():
    import torch
    t = torch.arange(24, dtype=torch.float32).reshape(2, 3, 4)
    b = runtime.Buffer.from_tensor(t)
    assert not b.on_device and b.raw.host == t.data_ptr() and b.raw.device == 0
    assert b.shape == (2, 3, 4) and b.dtype == np.float32 and b.raw.dimensions == 3
    assert [(b.dims[i].extent, b.dims[i].stride) for i in range(3)] == [(4, 1), (3, 4), (2, 12)]     # innermost first
    assert runtime.Buffer.from_tensor(torch.zeros(5, dtype=torch.bfloat16)).dtype == np.uint16         # p_bfloat16 storage
    assert runtime.Buffer.from_tensor(torch.zeros(5, dtype=torch.int32)).raw.type.code == 0
    with pytest.raises(ValueError):
        runtime.Buffer.from_tensor(t.transpose(0, 2))


@pytest.mark.gpu
def test_sgemm_on_gpu_tensors_default_and_side_stream():
    import torch
    M, N, K = 128, 192, 96
    prog = runtime.load(PROGRAMS, "sgemm_%dx%dx%d" % (M, N, K))
    g = torch.Generator().manual_seed(3)
    A = torch.randint(-5, 5, (M, K), generator=g).float()
    B = torch.randint(-5, 5, (K, N), generator=g).float()
    C = torch.randint(-5, 5, (M, N), generator=g).float()
    scal = np.array([3.0, 2.0], np.float32)
    expected = 3.0 * (A.double() @ B.double()) + 2.0 * C.double()
    # torch's default stream: the call waits on both sides
    dA, dB, dC = A.cuda(), B.cuda(), C.cuda()
    print("default stream", flush=True)
    prog(scal, dA, dB, dC)
    assert torch.equal(dC.cpu().double(), expected)
    # a side stream: the function's kernels are ordered between torch kernels of that stream
    side = torch.cuda.Stream()
    before = runtime.wrappers().tiramisu_hip_get_stream()
    print("side stream", flush=True)
    with torch.cuda.stream(side):
        dA2 = (A.cuda(non_blocking=True) * 2.0)          # produced on the side stream just before the call
        dC2 = C.cuda(non_blocking=True) + 0.0
        prog(scal, dA2, dB, dC2)
        result = dC2 * 1.0                               # consumed on the side stream right after
    side.synchronize()
    assert torch.equal(result.cpu().double(), 3.0 * (2.0 * A.double() @ B.double()) + 2.0 * C.double())
    assert runtime.wrappers().tiramisu_hip_get_stream() == before
    # a tensor in the wrong memory is refused before anything is launched
    with pytest.raises(ValueError):
        prog(scal, A, dB, dC)


@pytest.mark.gpu
def test_bf16_tensors_are_p_bfloat16_buffers():
    import torch
    M, N, K = 128, 192, 128
    name = "sgemm_bf16_%dx%dx%d" % (M, N, K)
    prog = runtime.load(PROGRAMS, name)
    g = torch.Generator().manual_seed(5)
    A = torch.randint(-4, 5, (M, K), generator=g).to(torch.bfloat16)
    B = torch.randint(-4, 5, (K, N), generator=g).to(torch.bfloat16)
    C = torch.zeros((M, N), dtype=torch.float32)
    dC = C.cuda()
    print(name, flush=True)
    prog(np.array([1.0, 0.0], np.float32), A.cuda(), B.cuda(), dC)
    assert torch.equal(dC.cpu().double(), A.double() @ B.double())
