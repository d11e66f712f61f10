"""Minimal ctypes view of the HIP runtime for timing and device copies
(events on a given stream, device-to-device copies, stream capture into a
graph). Used by the benchmark and the smoke check; the library itself links
the runtime directly."""
import ctypes as C

_rt = None


def rt():
    global _rt
    if _rt is None:
        _rt = C.CDLL("libamdhip64.so")
        _rt.hipGetErrorString.restype = C.c_char_p
    return _rt


def check(code, what):
    if code != 0:
        raise RuntimeError("%s: %s" % (what, rt().hipGetErrorString(code).decode()))


class Event:
    def __init__(self):
        self.h = C.c_void_p()
        check(rt().hipEventCreate(C.byref(self.h)), "hipEventCreate")

    def record(self, stream):
        check(rt().hipEventRecord(self.h, C.c_void_p(stream)), "hipEventRecord")

    def synchronize(self):
        check(rt().hipEventSynchronize(self.h), "hipEventSynchronize")

    def elapsed_ms(self, start):
        ms = C.c_float()
        check(rt().hipEventElapsedTime(C.byref(ms), start.h, self.h), "hipEventElapsedTime")
        return ms.value

    def __del__(self):
        if self.h:
            rt().hipEventDestroy(self.h)
            self.h = None


def malloc(nbytes):
    p = C.c_void_p()
    check(rt().hipMalloc(C.byref(p), C.c_size_t(nbytes)), "hipMalloc")
    return p.value


def free(ptr):
    check(rt().hipFree(C.c_void_p(ptr)), "hipFree")


def memset(ptr, byte, nbytes):
    check(rt().hipMemset(C.c_void_p(ptr), C.c_int(byte), C.c_size_t(nbytes)), "hipMemset")


def memcpy_dtod(dst, src, nbytes):
    check(rt().hipMemcpy(C.c_void_p(dst), C.c_void_p(src), C.c_size_t(nbytes), 3), "hipMemcpy")


def device_synchronize():
    check(rt().hipDeviceSynchronize(), "hipDeviceSynchronize")


def device_name():
    # hipDeviceProp_t is large; the name is its first field
    buf = C.create_string_buffer(4096)
    check(rt().hipGetDevicePropertiesR0600(buf, 0), "hipGetDeviceProperties")
    return buf.value.decode(errors="replace")


class Graph:
    """Capture whatever `fn` enqueues on `stream` and replay it."""

    def __init__(self, stream, fn):
        s = C.c_void_p(stream)
        check(rt().hipStreamBeginCapture(s, 0), "hipStreamBeginCapture")  # global mode
        try:
            fn()
        finally:
            g = C.c_void_p()
            code = rt().hipStreamEndCapture(s, C.byref(g))
        check(code, "hipStreamEndCapture")
        self.graph = g
        self.exe = C.c_void_p()
        check(rt().hipGraphInstantiate(C.byref(self.exe), g, None, None, 0), "hipGraphInstantiate")
        self.stream = stream

    def launch(self):
        check(rt().hipGraphLaunch(self.exe, C.c_void_p(self.stream)), "hipGraphLaunch")

    def __del__(self):
        if getattr(self, "exe", None):
            rt().hipGraphExecDestroy(self.exe)
            rt().hipGraphDestroy(self.graph)
            self.exe = None
