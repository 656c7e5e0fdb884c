"""Minimal ctypes view of the HIP runtime: device memory, streams, events.

Used by the tests and the bench to own device buffers and to time launches on
the stream the kernels run on.  It binds the same libamdhip64 the C-ABI library
is linked against, so there is exactly one HIP runtime in the process.
"""
import ctypes as C

import numpy as np

_rt = None

hipMemcpyHostToDevice = 1
hipMemcpyDeviceToHost = 2
hipMemcpyDeviceToDevice = 3


class HipError(RuntimeError):
    pass


def rt():
    global _rt
    if _rt is None:
        last = None
        for name in ("libamdhip64.so.7", "libamdhip64.so", "/opt/rocm/lib/libamdhip64.so"):
            try:
                _rt = C.CDLL(name, mode=C.RTLD_GLOBAL)
                break
            except OSError as e:  # pragma: no cover - depends on the box
                last = e
        if _rt is None:
            raise HipError(f"cannot load the HIP runtime: {last}")
        _rt.hipGetErrorString.restype = C.c_char_p
        _rt.hipGetErrorString.argtypes = [C.c_int]
    return _rt


def check(code, what=""):
    if code != 0:
        msg = rt().hipGetErrorString(code)
        raise HipError(f"{what}: HIP error {code}: {msg.decode() if msg else '?'}")


def device_count():
    n = C.c_int(0)
    try:
        code = rt().hipGetDeviceCount(C.byref(n))
    except HipError:
        return 0
    return n.value if code == 0 else 0


def set_device(i):
    check(rt().hipSetDevice(C.c_int(i)), "hipSetDevice")


def synchronize():
    check(rt().hipDeviceSynchronize(), "hipDeviceSynchronize")


def device_name():
    """Marketing name of device 0, with its architecture name when the runtime reports one
    (hipGetDeviceProperties: `name` is the first field of the struct, `gcnArchName` a later one that
    is found by its "gfx" prefix, so no struct layout is assumed)."""
    buf = C.create_string_buffer(8192)
    fn = getattr(rt(), "hipGetDevicePropertiesR0600", None) or rt().hipGetDeviceProperties
    name, arch = "", ""
    if fn(buf, C.c_int(0)) == 0:
        raw = buf.raw
        name = raw[:256].split(b"\0", 1)[0].decode(errors="replace")
        at = raw.find(b"gfx", 256)
        if at >= 0:
            arch = raw[at:at + 64].split(b"\0", 1)[0].decode(errors="replace")
    if not name:
        short = C.create_string_buffer(256)
        if rt().hipDeviceGetName(short, C.c_int(256), C.c_int(0)) == 0:
            name = short.value.decode(errors="replace")
    return " ".join(x for x in (name, arch) if x) or "unknown HIP device"


class DeviceBuffer:
    """Owning device allocation."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self._ptr = C.c_void_p(0)
        check(rt().hipMalloc(C.byref(self._ptr), C.c_size_t(max(self.nbytes, 1))), "hipMalloc")

    @property
    def ptr(self):
        return self._ptr.value

    def at(self, offset):
        return C.c_void_p(self._ptr.value + int(offset))

    def free(self):
        if self._ptr is not None and self._ptr.value:
            rt().hipFree(self._ptr)
            self._ptr = C.c_void_p(0)

    def __del__(self):
        try:
            self.free()
        except Exception:  # interpreter shutdown
            pass

    # -- transfers (synchronous) --
    def upload(self, arr, offset=0):
        a = np.ascontiguousarray(arr)
        assert offset + a.nbytes <= self.nbytes, "upload past the end of the buffer"
        if a.nbytes:
            check(rt().hipMemcpy(self.at(offset), a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes),
                                 C.c_int(hipMemcpyHostToDevice)), "hipMemcpy H2D")
        return self

    def download(self, dtype, count=None, offset=0):
        dtype = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset) // dtype.itemsize
        out = np.empty(count, dtype)
        assert offset + out.nbytes <= self.nbytes, "download past the end of the buffer"
        if out.nbytes:
            check(rt().hipMemcpy(out.ctypes.data_as(C.c_void_p), self.at(offset), C.c_size_t(out.nbytes),
                                 C.c_int(hipMemcpyDeviceToHost)), "hipMemcpy D2H")
        return out

    def fill(self, byte=0):
        check(rt().hipMemset(self._ptr, C.c_int(byte), C.c_size_t(self.nbytes)), "hipMemset")
        return self


def to_device(arr):
    a = np.ascontiguousarray(arr)
    return DeviceBuffer(a.nbytes).upload(a)


class Stream:
    def __init__(self):
        self._s = C.c_void_p(0)
        check(rt().hipStreamCreate(C.byref(self._s)), "hipStreamCreate")

    @property
    def handle(self):
        return self._s

    def synchronize(self):
        check(rt().hipStreamSynchronize(self._s), "hipStreamSynchronize")

    def __del__(self):
        try:
            if self._s.value:
                rt().hipStreamDestroy(self._s)
        except Exception:
            pass


class Graph:
    """A stream capture turned into an executable graph: with Graph(stream): ...launches...; then
    graph.launch() replays them on that stream."""

    def __init__(self, stream):
        self._stream = stream
        self._graph = C.c_void_p(0)
        self._exec = C.c_void_p(0)

    def __enter__(self):
        check(rt().hipStreamBeginCapture(self._stream.handle, 1), "hipStreamBeginCapture")   # thread-local mode
        return self

    def __exit__(self, exc_type, exc, tb):
        code = rt().hipStreamEndCapture(self._stream.handle, C.byref(self._graph))
        if exc_type is None:
            check(code, "hipStreamEndCapture")
            check(rt().hipGraphInstantiate(C.byref(self._exec), self._graph, None, None, C.c_size_t(0)),
                  "hipGraphInstantiate")
        return False

    def launch(self):
        check(rt().hipGraphLaunch(self._exec, self._stream.handle), "hipGraphLaunch")

    def __del__(self):
        try:
            if self._exec.value:
                rt().hipGraphExecDestroy(self._exec)
            if self._graph.value:
                rt().hipGraphDestroy(self._graph)
        except Exception:
            pass


class Event:
    def __init__(self):
        self._e = C.c_void_p(0)
        check(rt().hipEventCreate(C.byref(self._e)), "hipEventCreate")

    def record(self, stream=None):
        s = stream.handle if stream is not None else C.c_void_p(0)
        check(rt().hipEventRecord(self._e, s), "hipEventRecord")

    def synchronize(self):
        check(rt().hipEventSynchronize(self._e), "hipEventSynchronize")

    def elapsed_ms(self, end):
        ms = C.c_float(0)
        check(rt().hipEventElapsedTime(C.byref(ms), self._e, end._e), "hipEventElapsedTime")
        return ms.value

    def __del__(self):
        try:
            if self._e.value:
                rt().hipEventDestroy(self._e)
        except Exception:
            pass
