"""Device buffers for tests through the HIP runtime itself (ctypes on libamdhip64), so that tests
of the device-pointer entry points need nothing but the library under test and the runtime."""
import ctypes as C

import numpy as np

_hip = None


def hip():
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so")
        _hip.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        _hip.hipFree.argtypes = [C.c_void_p]
        _hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _hip.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
    return _hip


def mem_free() -> int:
    """Free device memory in bytes as the runtime reports it (hipMemGetInfo)."""
    free, total = C.c_size_t(), C.c_size_t()
    rc = hip().hipDeviceSynchronize() or hip().hipMemGetInfo(C.byref(free), C.byref(total))
    if rc:
        raise RuntimeError(f"hipMemGetInfo failed: {rc}")
    return free.value


class DeviceArray:
    """A device allocation with a NumPy dtype/shape; `.ptr` is the raw device pointer."""

    def __init__(self, shape, dtype, fill=None):
        self.shape, self.dtype = tuple(shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = C.c_void_p()
        rc = hip().hipMalloc(C.byref(p), max(self.nbytes, 4))
        if rc:
            raise RuntimeError(f"hipMalloc failed: {rc}")
        self.ptr = p.value
        if fill is not None:
            hip().hipMemset(self.ptr, fill, self.nbytes)

    @classmethod
    def from_host(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        rc = hip().hipMemcpy(d.ptr, a.ctypes.data, a.nbytes, 1)  # hipMemcpyHostToDevice
        if rc:
            raise RuntimeError(f"hipMemcpy H2D failed: {rc}")
        return d

    def to_host(self):
        out = np.empty(self.shape, self.dtype)
        rc = hip().hipDeviceSynchronize()
        rc = rc or hip().hipMemcpy(out.ctypes.data, self.ptr, self.nbytes, 2)  # DeviceToHost
        if rc:
            raise RuntimeError(f"hipMemcpy D2H failed: {rc}")
        return out

    def free(self):
        if self.ptr:
            hip().hipFree(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    """A HIP stream created through the runtime (default priority)."""

    def __init__(self):
        h = hip()
        h.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
        h.hipStreamDestroy.argtypes = [C.c_void_p]
        h.hipStreamSynchronize.argtypes = [C.c_void_p]
        p = C.c_void_p()
        rc = h.hipStreamCreate(C.byref(p))
        if rc:
            raise RuntimeError(f"hipStreamCreate failed: {rc}")
        self.ptr = p.value

    def synchronize(self):
        rc = hip().hipStreamSynchronize(self.ptr)
        if rc:
            raise RuntimeError(f"hipStreamSynchronize failed: {rc}")

    def close(self):
        if self.ptr:
            hip().hipStreamDestroy(self.ptr)
            self.ptr = None


class Graph:
    """Capture of the work launched on a stream between begin() and end(), replayable."""

    def __init__(self, stream):
        h = hip()
        h.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        h.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        h.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p,
                                          C.c_size_t]
        h.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        h.hipGraphExecDestroy.argtypes = [C.c_void_p]
        h.hipGraphDestroy.argtypes = [C.c_void_p]
        self.stream, self.graph, self.exe = stream, C.c_void_p(), C.c_void_p()

    def begin(self):
        rc = hip().hipStreamBeginCapture(self.stream.ptr, 0)  # hipStreamCaptureModeGlobal
        if rc:
            raise RuntimeError(f"hipStreamBeginCapture failed: {rc}")

    def end(self):
        rc = hip().hipStreamEndCapture(self.stream.ptr, C.byref(self.graph))
        rc = rc or hip().hipGraphInstantiate(C.byref(self.exe), self.graph, None, None, 0)
        if rc:
            raise RuntimeError(f"graph capture / instantiate failed: {rc}")

    def launch(self):
        rc = hip().hipGraphLaunch(self.exe, self.stream.ptr)
        if rc:
            raise RuntimeError(f"hipGraphLaunch failed: {rc}")

    def close(self):
        if self.exe:
            hip().hipGraphExecDestroy(self.exe)
            hip().hipGraphDestroy(self.graph)
            self.exe = None
