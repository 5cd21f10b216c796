"""Device memory for the engine: a hipMalloc-backed buffer with Storage-like ownership
(the slot of `Storage::Cuda`, crates/rustorch-core/src/tensor/storage.rs:776-817; the pattern
of the wgpu payload, :538-644: freed exactly once, on last drop)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib as L
from .errors import raise_for


class HipStorage:
    """Owns `byte_len` bytes of HBM.  `ptr` is the raw device address (what the FFI takes)."""

    def __init__(self, byte_len: int):
        err = L.RtErr()
        self.byte_len = int(byte_len)
        self.ptr = L.lib().rt_buf_alloc(self.byte_len, C.byref(err))
        if not self.ptr:
            raise_for(L.RT_ERR_HIP if err.hip_error else L.RT_ERR_NO_DEVICE, err)

    @classmethod
    def from_numpy(cls, a: np.ndarray, stream=None) -> "HipStorage":
        a = np.ascontiguousarray(a)
        s = cls(a.nbytes)
        s.upload(a, stream)
        return s

    @classmethod
    def zeros(cls, byte_len: int, stream=None) -> "HipStorage":
        """A zero-filled buffer (byte_len a multiple of 4); the fill is enqueued on `stream`."""
        s = cls(byte_len)
        err = L.RtErr()
        raise_for(L.lib().rt_buf_zero(s.ptr, s.byte_len, stream, C.byref(err)), err)
        return s

    def upload(self, a: np.ndarray, stream=None):
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.byte_len
        err = L.RtErr()
        raise_for(L.lib().rt_memcpy_h2d(self.ptr, a.ctypes.data, a.nbytes, stream, C.byref(err)), err)
        synchronize(stream)

    def download(self, dtype, count=None, stream=None) -> np.ndarray:
        dtype = np.dtype(dtype)
        n = self.byte_len // dtype.itemsize if count is None else count
        out = np.empty(n, dtype=dtype)
        err = L.RtErr()
        raise_for(L.lib().rt_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes, stream, C.byref(err)), err)
        synchronize(stream)
        return out

    def free(self):
        if getattr(self, "ptr", None):
            err = L.RtErr()
            L.lib().rt_buf_free(self.ptr, C.byref(err))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def synchronize(stream=None):
    err = L.RtErr()
    raise_for(L.lib().rt_stream_synchronize(stream, C.byref(err)), err)


class Stream:
    """A HIP stream at the default priority; pass `.handle` (or the object) as the `stream` of a device entry."""

    def __init__(self):
        err = L.RtErr()
        self.handle = L.lib().rt_stream_create(C.byref(err))
        if not self.handle:
            raise_for(L.RT_ERR_HIP if err.hip_error else L.RT_ERR_NO_DEVICE, err)

    @property
    def _as_parameter_(self):  # lets ctypes take the object where a void* is expected
        return C.c_void_p(self.handle)

    def synchronize(self):
        synchronize(self.handle)

    def destroy(self):
        if getattr(self, "handle", None):
            err = L.RtErr()
            L.lib().rt_stream_destroy(self.handle, C.byref(err))
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def init(device: int = 0):
    """Select the gfx950 device; raises DeviceError(NoDeviceFound) when there is none."""
    err = L.RtErr()
    raise_for(L.lib().rt_init(device, C.byref(err)), err)


def shutdown():
    """Free the buffers the library keeps between calls (it stays usable; they come back on demand)."""
    err = L.RtErr()
    raise_for(L.lib().rt_shutdown(C.byref(err)), err)


def i32_add_dev(buf, n: int, delta: int, stream=None):
    """Adds `delta` to the `n` int32 values of a device buffer, asynchronously on `stream` (positions and context
    lengths of a decode loop that lives in a HIP graph)."""
    err = L.RtErr()
    raise_for(L.lib().rt_i32_add_dev(stream, dev_ptr(buf), n, delta, C.byref(err)), err)


def debug_force_bf16_prefill_kernel(name: str = "auto"):
    """Measurement / test switch: "auto", "tile" or "persistent" for the bf16 prefill entries."""
    rc = L.lib().rt_debug_force_bf16_prefill_kernel({"auto": 0, "tile": 1, "persistent": 2, "wide": 3}[name])
    if rc:
        raise ValueError(name)


def set_strict_non_finite_v(on: bool) -> bool:
    """Causal prefill entries follow the reference for non-finite V at hidden keys (every row NaN in that column,
    cpu_forward.rs:268-425) at the cost of one more pass over V.  Returns the previous setting."""
    return bool(L.lib().rt_set_strict_non_finite_v(1 if on else 0))


def dev_ptr(x) -> int:
    """Raw device address of a HipStorage, a torch tensor on the GPU, or an int."""
    if x is None:
        return None
    if isinstance(x, HipStorage):
        return x.ptr
    if isinstance(x, (int, np.integer)):
        return int(x)
    if hasattr(x, "data_ptr"):
        assert x.is_cuda and x.is_contiguous(), "device entry points take contiguous GPU tensors"
        return x.data_ptr()
    raise TypeError(type(x))
