"""Minimal ctypes binding of the HIP runtime: device memory copies, streams and events.
Used by tests and the benchmark for plumbing only."""
import ctypes as C

_hip = None


class HipError(RuntimeError):
    pass


def lib():
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so", mode=C.RTLD_GLOBAL)
        _hip.hipGetErrorString.restype = C.c_char_p
    return _hip


def check(code, what=""):
    if code != 0:
        raise HipError("%s: HIP error %d (%s)" % (what, code, lib().hipGetErrorString(code).decode()))


H2D, D2H, D2D = 1, 2, 3


def device_count():
    n = C.c_int(0)
    code = lib().hipGetDeviceCount(C.byref(n))
    return n.value if code == 0 else 0


def synchronize():
    check(lib().hipDeviceSynchronize(), "hipDeviceSynchronize")


def memcpy(dst, src, nbytes, kind):
    check(lib().hipMemcpy(C.c_void_p(dst), C.c_void_p(src), C.c_size_t(nbytes), C.c_int(kind)),
          "hipMemcpy")


def memset(dst, value, nbytes):
    check(lib().hipMemset(C.c_void_p(dst), C.c_int(value), C.c_size_t(nbytes)), "hipMemset")


def upload(dst, array):
    """numpy array (C-contiguous) -> device address."""
    memcpy(dst, array.ctypes.data, array.nbytes, H2D)


def download(array, src):
    """device address -> numpy array (C-contiguous, preallocated)."""
    memcpy(array.ctypes.data, src, array.nbytes, D2H)


def malloc(nbytes):
    p = C.c_void_p()
    check(lib().hipMalloc(C.byref(p), C.c_size_t(nbytes)), "hipMalloc")
    return p.value


def free(ptr):
    check(lib().hipFree(C.c_void_p(ptr)), "hipFree")


class Stream:
    def __init__(self):
        self.handle = C.c_void_p()
        check(lib().hipStreamCreate(C.byref(self.handle)), "hipStreamCreate")

    @property
    def ptr(self):
        return self.handle.value

    def synchronize(self):
        check(lib().hipStreamSynchronize(self.handle), "hipStreamSynchronize")

    def destroy(self):
        if self.handle:
            lib().hipStreamDestroy(self.handle)
            self.handle = C.c_void_p()


class Event:
    def __init__(self):
        self.handle = C.c_void_p()
        check(lib().hipEventCreate(C.byref(self.handle)), "hipEventCreate")

    def record(self, stream=None):
        s = stream.handle if stream is not None else C.c_void_p()
        check(lib().hipEventRecord(self.handle, s), "hipEventRecord")

    def synchronize(self):
        check(lib().hipEventSynchronize(self.handle), "hipEventSynchronize")

    def elapsed_ms(self, end):
        ms = C.c_float(0)
        check(lib().hipEventElapsedTime(C.byref(ms), self.handle, end.handle), "hipEventElapsedTime")
        return ms.value

    def destroy(self):
        if self.handle:
            lib().hipEventDestroy(self.handle)
            self.handle = C.c_void_p()


class Graph:
    """Stream capture into a HIP graph: `with Graph(stream) as g: ...enqueue...`, then g.launch()."""

    def __init__(self, stream):
        self.stream = stream
        self.graph = C.c_void_p()
        self.exe = C.c_void_p()

    def __enter__(self):
        # hipStreamCaptureModeThreadLocal = 1
        check(lib().hipStreamBeginCapture(self.stream.handle, C.c_int(1)), "hipStreamBeginCapture")
        return self

    def __exit__(self, exc_type, exc, tb):
        code = lib().hipStreamEndCapture(self.stream.handle, C.byref(self.graph))
        if exc_type is None:
            check(code, "hipStreamEndCapture")
            check(lib().hipGraphInstantiate(C.byref(self.exe), self.graph, None, None, C.c_size_t(0)),
                  "hipGraphInstantiate")

    def launch(self):
        check(lib().hipGraphLaunch(self.exe, self.stream.handle), "hipGraphLaunch")

    def destroy(self):
        if self.exe:
            lib().hipGraphExecDestroy(self.exe)
            self.exe = C.c_void_p()
        if self.graph:
            lib().hipGraphDestroy(self.graph)
            self.graph = C.c_void_p()
