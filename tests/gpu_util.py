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
