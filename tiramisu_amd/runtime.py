"""Calling compiled Tiramisu functions from Python through their C ABI.

A compiled Tiramisu function is ``extern "C" int f(halide_buffer_t *arg0, ...)``
(reference: the generated headers, e.g. tests/wrapper_test_167.h, and the buffer layout at
benchmarks/linear_algebra/blas/level1/dot/generated_dot.o.h:1157-1219).  This module is the
Python counterpart of the reference's C++ wrapper programs: it describes numpy arrays (host
memory) or raw device pointers as ``halide_buffer_t`` and calls the function with ctypes.
It contains no compute of its own and has no CPU fallback: loading fails loudly when the
HIP libraries were not built.
"""
import ctypes
import os

import numpy as np

from . import build as _build


class halide_dimension_t(ctypes.Structure):
    _fields_ = [("min", ctypes.c_int32), ("extent", ctypes.c_int32), ("stride", ctypes.c_int32),
                ("flags", ctypes.c_uint32)]


class halide_type_t(ctypes.Structure):
    _fields_ = [("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16)]


class halide_buffer_t(ctypes.Structure):
    _fields_ = [("device", ctypes.c_uint64), ("device_interface", ctypes.c_void_p),
                ("host", ctypes.c_void_p), ("flags", ctypes.c_uint64), ("type", halide_type_t),
                ("dimensions", ctypes.c_int32), ("dim", ctypes.POINTER(halide_dimension_t)),
                ("padding", ctypes.c_void_p)]


_TYPE_CODES = {"i": 0, "u": 1, "f": 2, "b": 1}


class Buffer:
    """Owns the ``halide_buffer_t`` (and its dimension array) describing one argument.

    Dimensions are stored innermost first, as Halide does: a C-contiguous numpy array of shape
    (M, N) has dim[0] = N (stride 1) and dim[1] = M (stride N)."""

    def __init__(self, shape, dtype, host_ptr=0, device_ptr=0, keepalive=None):
        dtype = np.dtype(dtype)
        self.keepalive = keepalive
        self.shape, self.dtype, self.on_device = tuple(int(v) for v in shape), dtype, bool(device_ptr)
        nd = len(shape)
        self.dims = (halide_dimension_t * max(nd, 1))()
        stride = 1
        for i, extent in enumerate(reversed(shape)):
            self.dims[i] = halide_dimension_t(0, int(extent), stride, 0)
            stride *= int(extent)
        self.raw = halide_buffer_t()
        self.raw.device = device_ptr
        self.raw.device_interface = None
        self.raw.host = host_ptr
        self.raw.flags = 0
        self.raw.type = halide_type_t(_TYPE_CODES[dtype.kind], dtype.itemsize * 8, 1)
        self.raw.dimensions = nd
        self.raw.dim = ctypes.cast(self.dims, ctypes.POINTER(halide_dimension_t))

    @staticmethod
    def from_numpy(a):
        if not a.flags["C_CONTIGUOUS"]:
            raise ValueError("Tiramisu buffers are dense row-major: pass a C-contiguous array")
        return Buffer(a.shape, a.dtype, host_ptr=a.ctypes.data, keepalive=a)

    @staticmethod
    def from_device(ptr, shape, dtype, keepalive=None):
        """A buffer that already lives in GPU memory (an argument tagged tag_gpu_global())."""
        return Buffer(shape, dtype, host_ptr=0, device_ptr=int(ptr), keepalive=keepalive)

    @staticmethod
    def from_tensor(t):
        """A ``torch.Tensor`` as an argument, without a copy: a tensor on the GPU describes a buffer tagged
        tag_gpu_global() (its storage is the device pointer), a CPU tensor a host buffer.  bfloat16 tensors
        are the 16-bit storage of p_bfloat16 buffers.  The tensor stays referenced while the buffer lives."""
        import torch
        if not t.is_contiguous():
            raise ValueError("Tiramisu buffers are dense row-major: pass a contiguous tensor")
        if t.dtype == torch.bfloat16:
            dtype = np.dtype(np.uint16)
        else:
            dtype = np.dtype(str(t.dtype).replace("torch.", ""))
        if t.is_cuda:
            return Buffer(tuple(t.shape), dtype, device_ptr=t.data_ptr(), keepalive=t)
        return Buffer(tuple(t.shape), dtype, host_ptr=t.data_ptr(), keepalive=t)

    def pointer(self):
        return ctypes.byref(self.raw)


_wrappers = None


def wrappers():
    """The runtime C ABI (include/tiramisu_hip_wrappers.h), loaded with global symbol visibility
    so that program libraries resolve against it."""
    global _wrappers
    if _wrappers is None:
        path = _build.wrappers_library()
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: run __graft_entry__.build() first" % path)
        lib = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
        lib.tiramisu_hip_malloc.restype = ctypes.c_void_p
        lib.tiramisu_hip_malloc.argtypes = [ctypes.c_uint64]
        lib.tiramisu_hip_free.argtypes = [ctypes.c_void_p]
        for fn in (lib.tiramisu_hip_memcpy_to_device, lib.tiramisu_hip_memcpy_to_host,
                   lib.tiramisu_hip_memcpy_device_to_device):
            fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64]
        lib.tiramisu_hip_stream_synchronize.argtypes = [ctypes.c_int32]
        lib.tiramisu_hip_set_stream.argtypes = [ctypes.c_void_p]
        lib.tiramisu_hip_get_stream.restype = ctypes.c_void_p
        lib.tiramisu_hip_stream_create.restype = ctypes.c_void_p
        lib.tiramisu_hip_stream_destroy.argtypes = [ctypes.c_void_p]
        lib.tiramisu_hip_sgemm_workspace.restype = ctypes.c_void_p
        lib.tiramisu_hip_kept_scratch.restype = ctypes.c_void_p
        lib.tiramisu_hip_kept_scratch.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.POINTER(ctypes.c_int32)]
        lib.tiramisu_hip_release_cached_memory.restype = ctypes.c_uint64
        lib.tiramisu_hip_cached_memory_bytes.restype = ctypes.c_uint64
        lib.tiramisu_hip_event_create.restype = ctypes.c_void_p
        lib.tiramisu_hip_event_record.argtypes = [ctypes.c_void_p]
        lib.tiramisu_hip_event_elapsed_ms.restype = ctypes.c_float
        lib.tiramisu_hip_event_elapsed_ms.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        lib.tiramisu_hip_event_destroy.argtypes = [ctypes.c_void_p]
        lib.tiramisu_hip_profile_name.restype = ctypes.c_char_p
        lib.tiramisu_hip_profile_name.argtypes = [ctypes.c_int]
        lib.tiramisu_hip_profile_ms.restype = ctypes.c_float
        lib.tiramisu_hip_profile_ms.argtypes = [ctypes.c_int]
        u64 = ctypes.c_uint64
        lib.tiramisu_hip_sgemm.argtypes = [ctypes.c_void_p] * 3 + [u64] * 3 + [ctypes.c_float] * 2 + \
            [u64] * 6 + [ctypes.c_bool] * 2
        lib.tiramisu_hip_sgemm_static_scratch.argtypes = lib.tiramisu_hip_sgemm.argtypes
        lib.tiramisu_hip_dgemm.argtypes = [ctypes.c_void_p] * 3 + [u64] * 3 + [ctypes.c_double] * 2 + \
            [u64] * 6 + [ctypes.c_bool] * 2
        _wrappers = lib
    return _wrappers


_C_TYPES = {"float": "float32", "double": "float64", "int8_t": "int8", "int16_t": "int16", "int32_t": "int32", "int64_t": "int64",
            "uint8_t": "uint8", "uint16_t": "uint16", "uint32_t": "uint32", "uint64_t": "uint64", "bool": "bool",
            "tiramisu_bf16_t": "uint16"}


def manifest_of(library_path, function_name):
    """The description the HIP back-end writes next to each object (``<object>.json``: arguments
    with type, shape and memory space, kernels emitted) for the object that ``lib<stem>.so`` was
    linked from (``<stem>.o`` or ``generated_fct_<stem>.o`` in the same directory), or None."""
    import json
    directory, base = os.path.split(os.path.abspath(library_path))
    stem = base[3:-3] if base.startswith("lib") and base.endswith(".so") else base
    for name in (stem + ".o.json", "generated_fct_" + stem + ".o.json"):
        path = os.path.join(directory, name)
        if os.path.exists(path):
            try:
                m = json.load(open(path))
            except ValueError:
                return None
            return m if m.get("function") == function_name else None
    return None


class Program:
    """One compiled Tiramisu function: ``Program(path, "test_167")(A, B, C)`` with numpy arrays
    and/or ``Buffer`` objects as arguments.  When the back-end's description of the function is
    found next to the library, arguments are checked against it before the call (count, element
    type, constant extents, host or device memory): a wrong buffer would otherwise be a
    out-of-bounds access on the GPU."""

    def __init__(self, library_path, function_name, needs_gpu_runtime=True):
        if not os.path.exists(library_path):
            raise RuntimeError("%s is missing: run __graft_entry__.build() first" % library_path)
        if needs_gpu_runtime:
            wrappers()
        self.lib = ctypes.CDLL(library_path)
        self.fn = getattr(self.lib, function_name)
        self.fn.restype = ctypes.c_int
        self.name = function_name
        self.manifest = manifest_of(library_path, function_name) if needs_gpu_runtime else None

    def check(self, bufs):
        expected = self.manifest["arguments"]
        if len(bufs) != len(expected):
            raise ValueError("%s takes %d buffers, %d given" % (self.name, len(expected), len(bufs)))
        for b, e in zip(bufs, expected):
            if np.dtype(_C_TYPES.get(e["type"], b.dtype)) != b.dtype:
                raise ValueError("%s: buffer %s holds %s, %s given" % (self.name, e["name"], e["type"], b.dtype))
            if (e["memory"] == "device") != b.on_device:
                raise ValueError("%s: buffer %s lives in %s memory" % (self.name, e["name"], e["memory"]))
            # a host input may be declared larger than what the program reads of it (the reference's
            # sgemm generators declare their two scalars over the row range); anything the GPU
            # touches, and every output, must have the declared number of elements
            strict = e["memory"] == "device" or e["kind"] != "input"
            if strict and all(isinstance(v, int) for v in e["shape"]):
                want = int(np.prod(e["shape"])) if e["shape"] else 1
                if int(np.prod(b.shape)) != want:
                    raise ValueError("%s: buffer %s has shape %s, %s given" % (self.name, e["name"], e["shape"], list(b.shape)))

    def __call__(self, *args):
        """Arguments: ``Buffer`` objects, numpy arrays (host buffers) or torch tensors (host or GPU buffers by where
        they live).  With a GPU tensor among them the function's kernels run on torch's current stream of that
        tensor's device, in order with the torch work around the call (the runtime's stream of the calling thread is
        put back afterwards); when that is torch's default stream the call waits for it first and for its own
        kernels afterwards."""
        bufs, torch_stream = [], None
        for a in args:
            if isinstance(a, Buffer):
                bufs.append(a)
            elif isinstance(a, np.ndarray):
                bufs.append(Buffer.from_numpy(a))
            elif type(a).__module__.split(".")[0] == "torch":
                bufs.append(Buffer.from_tensor(a))
                if a.is_cuda and torch_stream is None:
                    import torch
                    torch_stream = torch.cuda.current_stream(a.device).cuda_stream
            else:
                bufs.append(Buffer.from_numpy(a))
        if self.manifest is not None:
            self.check(bufs)
        if torch_stream is None:
            rc = self.fn(*[b.pointer() for b in bufs])
        elif torch_stream == 0:
            # torch's default stream is the device's null stream, which the runtime has no handle for: order the
            # call by waiting on both sides instead
            import torch
            torch.cuda.current_stream().synchronize()
            rc = self.fn(*[b.pointer() for b in bufs])
            wrappers().tiramisu_hip_stream_synchronize(0)
        else:
            w = wrappers()
            before = w.tiramisu_hip_get_stream()
            w.tiramisu_hip_set_stream(torch_stream)
            try:
                rc = self.fn(*[b.pointer() for b in bufs])
            finally:
                w.tiramisu_hip_set_stream(before)
        if rc != 0:
            raise RuntimeError("Tiramisu function returned %d" % rc)
        return rc


def load(directory, name, function_name=None):
    return Program(_build.program_library(directory, name), function_name or name)


def profile(fn):
    """Run ``fn()`` with per-launch timing on; returns [(kernel name, milliseconds), ...]."""
    w = wrappers()
    w.tiramisu_hip_profile_start()
    fn()
    n = w.tiramisu_hip_profile_stop()
    return [(w.tiramisu_hip_profile_name(i).decode(), float(w.tiramisu_hip_profile_ms(i))) for i in range(n)]


class DeviceTimer:
    """HIP-event timing on the stream that generated code launches on."""

    def __init__(self):
        self.w = wrappers()
        self.start = self.w.tiramisu_hip_event_create()
        self.stop = self.w.tiramisu_hip_event_create()

    def __enter__(self):
        self.w.tiramisu_hip_event_record(self.start)
        return self

    def __exit__(self, *exc):
        self.w.tiramisu_hip_event_record(self.stop)
        self.ms = self.w.tiramisu_hip_event_elapsed_ms(self.start, self.stop)
        return False
