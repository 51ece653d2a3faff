"""Device buffers for the GPU tests, through the runtime C ABI only (no torch)."""
import numpy as np

from tiramisu_amd import runtime


class DeviceArray:
    def __init__(self, host):
        self.w = runtime.wrappers()
        self.shape, self.dtype, self.nbytes = host.shape, host.dtype, host.nbytes
        self.ptr = self.w.tiramisu_hip_malloc(max(self.nbytes, 16))
        self.upload(host)

    def upload(self, host):
        host = np.ascontiguousarray(host)
        self.w.tiramisu_hip_memcpy_to_device(self.ptr, host.ctypes.data, host.nbytes)

    def download(self):
        out = np.empty(self.shape, self.dtype)
        self.w.tiramisu_hip_stream_synchronize(0)
        self.w.tiramisu_hip_memcpy_to_host(out.ctypes.data, self.ptr, self.nbytes)
        return out

    def buffer(self):
        return runtime.Buffer.from_device(self.ptr, self.shape, self.dtype, keepalive=self)

    def free(self):
        if self.ptr:
            self.w.tiramisu_hip_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def assert_fp32_parity(out, ref, what, rtol=1e-4, atol=None):
    """The fp32 bar of the parity statement ("max relative error <= 1e-4"; 2e-2 for bf16 inputs), read two
    ways, both asserted and both printed:
      * normalised maximum norm:  max|out - ref| <= rtol * max|ref|;
      * element by element:       |out - ref| <= rtol * |ref| + atol  with  atol = rtol * rms(ref)
        (results are sums of many products, so an element near zero carries the rounding error of terms
        of the typical magnitude: the absolute allowance is rtol times that magnitude)."""
    r = np.asarray(ref, np.float64)
    d = np.abs(np.asarray(out, np.float64) - r)
    if atol is None:
        atol = rtol * float(np.sqrt(np.mean(r * r)))
    norm_err = float(d.max() / max(np.max(np.abs(r)), 1e-300))
    worst = float(np.max(d / (rtol * np.abs(r) + atol))) if atol > 0 else (0.0 if d.max() == 0 else np.inf)
    print("%s: max|d|/max|ref| = %.3g (bar %g); worst element |d|/(rtol*|ref|+atol) = %.3g (rtol %g, atol %.3g)"
          % (what, norm_err, rtol, worst, rtol, atol), flush=True)
    assert norm_err <= rtol, what
    assert worst <= 1.0, what
