"""Device buffers for the GPU tests of the `_dev` entry points, on the HIP runtime the product library itself
is linked against (one HIP runtime per process: a second one, such as the copy bundled with PyTorch, finds no
device once the first holds it)."""
import ctypes as C

import numpy as np

_hip = None


def hip():
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so.7")
        _hip.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        _hip.hipFree.argtypes = [C.c_void_p]
        _hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _hip.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        _hip.hipDeviceSynchronize.argtypes = []
        _hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    return _hip


def _ok(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed with HIP error {rc}")


def free_device_bytes():
    """Free device memory as hipMemGetInfo reports it (after a device synchronisation)."""
    _ok(hip().hipDeviceSynchronize(), "hipDeviceSynchronize")
    free, total = C.c_size_t(), C.c_size_t()
    _ok(hip().hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
    return free.value


class DevBuf:
    """nbytes of device memory; from_numpy / to_numpy copy synchronously."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        _ok(hip().hipMalloc(C.byref(p), max(self.nbytes, 8)), "hipMalloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        if a.nbytes:
            _ok(hip().hipMemcpy(b.ptr, a.ctypes.data_as(C.c_void_p), a.nbytes, 1), "hipMemcpy H2D")
        return b

    def to_numpy(self, shape, dtype=np.float64):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            _ok(hip().hipMemcpy(out.ctypes.data_as(C.c_void_p), self.ptr, out.nbytes, 2), "hipMemcpy D2H")
        return out

    def zero(self):
        _ok(hip().hipMemset(self.ptr, 0, self.nbytes), "hipMemset")

    def free(self):
        if self.ptr:
            hip().hipFree(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
