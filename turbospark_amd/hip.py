"""The handful of HIP runtime calls the host side needs (device buffers for drafter logits,
events on the engine's stream), bound with ctypes so no framework import is required."""
import ctypes as C

_rt = None


def rt():
    global _rt
    if _rt is None:
        L = C.CDLL("libamdhip64.so")
        L.hipGetErrorString.restype = C.c_char_p
        L.hipGetErrorString.argtypes = [C.c_int]
        L.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        L.hipFree.argtypes = [C.c_void_p]
        L.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        L.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        L.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        L.hipEventSynchronize.argtypes = [C.c_void_p]
        L.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        L.hipEventDestroy.argtypes = [C.c_void_p]
        L.hipStreamSynchronize.argtypes = [C.c_void_p]
        L.hipGetDeviceCount.argtypes = [C.POINTER(C.c_int)]
        _rt = L
    return _rt


def check(code, what):
    if code != 0:
        raise RuntimeError(f"{what}: {rt().hipGetErrorString(code).decode()}")


def device_count():
    n = C.c_int(0)
    try:
        if rt().hipGetDeviceCount(C.byref(n)) != 0:
            return 0
    except OSError:
        return 0
    return n.value


class DeviceBuffer:
    def __init__(self, nbytes):
        self.ptr = C.c_void_p()
        self.nbytes = nbytes
        check(rt().hipMalloc(C.byref(self.ptr), nbytes), "hipMalloc")

    def upload(self, array):
        assert array.nbytes <= self.nbytes
        check(rt().hipMemcpy(self.ptr, array.ctypes.data, array.nbytes, 1), "hipMemcpy H2D")
        return self

    def free(self):
        if self.ptr:
            rt().hipFree(self.ptr)
            self.ptr = C.c_void_p()

    def __del__(self):
        self.free()

    def address(self, byte_offset=0):
        return self.ptr.value + byte_offset


class Event:
    def __init__(self):
        self.h = C.c_void_p()
        check(rt().hipEventCreate(C.byref(self.h)), "hipEventCreate")

    def record(self, stream):
        check(rt().hipEventRecord(self.h, C.c_void_p(stream)), "hipEventRecord")

    def sync(self):
        check(rt().hipEventSynchronize(self.h), "hipEventSynchronize")

    def ms_since(self, earlier):
        t = C.c_float()
        check(rt().hipEventElapsedTime(C.byref(t), earlier.h, self.h), "hipEventElapsedTime")
        return t.value

    def __del__(self):
        if self.h:
            rt().hipEventDestroy(self.h)
