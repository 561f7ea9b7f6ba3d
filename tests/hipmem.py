"""Caller-owned device buffers for the operator-level tests, through the same HIP runtime the
library is linked against (ctypes on libamdhip64; PyTorch bundles a different copy of the runtime,
and two runtimes in one process do not share a device context)."""
import ctypes as C

import numpy as np

_hip = None


def hip():
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so.7")  # already mapped by libbnn_hmc.so: same handle
        _hip.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        _hip.hipFree.argtypes = [C.c_void_p]
        _hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _hip.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        _hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    return _hip


def _ok(rc, what):
    if rc != 0:
        raise RuntimeError("%s failed with hipError %d" % (what, rc))


class DevBuf:
    """A device allocation of `nbytes` bytes; `.ptr` is the device address as an int."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        _ok(hip().hipMalloc(C.byref(p), max(self.nbytes, 4)), "hipMalloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a, offset_bytes=0):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes + offset_bytes + 64)
        _ok(hip().hipMemcpy(b.ptr + offset_bytes, a.ctypes.data, a.nbytes, 1), "hipMemcpy H2D")
        b.data_ptr = b.ptr + offset_bytes
        return b

    @classmethod
    def full(cls, count, value, dtype=np.float32):
        return cls.from_numpy(np.full(count, value, dtype))

    def numpy(self, count, dtype=np.float32, offset_bytes=0):
        out = np.empty(count, dtype)
        _ok(hip().hipDeviceSynchronize(), "hipDeviceSynchronize")
        _ok(hip().hipMemcpy(out.ctypes.data, self.ptr + offset_bytes, out.nbytes, 2), "hipMemcpy D2H")
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


def free_bytes():
    """free device memory as the runtime reports it"""
    free, total = C.c_size_t(), C.c_size_t()
    _ok(hip().hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
    return free.value


def synchronize():
    _ok(hip().hipDeviceSynchronize(), "hipDeviceSynchronize")
