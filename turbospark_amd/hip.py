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
        L.hipStreamCreateWithFlags.argtypes = [C.POINTER(C.c_void_p), C.c_uint]
        L.hipStreamDestroy.argtypes = [C.c_void_p]
        L.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        L.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        L.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        L.hipGraphDestroy.argtypes = [C.c_void_p]
        L.hipGraphExecDestroy.argtypes = [C.c_void_p]
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


class Stream:
    """A non-blocking stream of the caller's own (graph capture needs one: the NULL stream cannot be captured)."""

    def __init__(self):
        self.h = C.c_void_p()
        check(rt().hipStreamCreateWithFlags(C.byref(self.h), 1), "hipStreamCreateWithFlags")

    def sync(self):
        check(rt().hipStreamSynchronize(self.h), "hipStreamSynchronize")

    def __del__(self):
        if self.h:
            rt().hipStreamDestroy(self.h)


class CapturedGraph:
    """What `record(stream)` enqueues on `stream`, captured once (thread-local mode) and replayable."""

    def __init__(self, stream, record):
        g = C.c_void_p()
        check(rt().hipStreamBeginCapture(stream.h, 1), "hipStreamBeginCapture")
        try:
            record(stream)
        finally:
            code = rt().hipStreamEndCapture(stream.h, C.byref(g))
        check(code, "hipStreamEndCapture")
        self.exe = C.c_void_p()
        code = rt().hipGraphInstantiate(C.byref(self.exe), g, None, None, 0)
        rt().hipGraphDestroy(g)
        check(code, "hipGraphInstantiate")
        self.stream = stream

    def launch(self):
        check(rt().hipGraphLaunch(self.exe, self.stream.h), "hipGraphLaunch")

    def __del__(self):
        if getattr(self, "exe", None):
            rt().hipGraphExecDestroy(self.exe)
