"""Minimal ctypes binding of the HIP runtime: device memory, copies, streams and
events for tests and bench.  Plumbing only -- no arithmetic happens here."""
import ctypes
import os

import numpy as np

_HIP = None

hipMemcpyHostToDevice = 1
hipMemcpyDeviceToHost = 2
hipMemcpyDeviceToDevice = 3
hipStreamNonBlocking = 1


class HipError(RuntimeError):
    pass


def lib():
    global _HIP
    if _HIP is None:
        last = None
        rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
        for name in ("libamdhip64.so", "libamdhip64.so.7", os.path.join(rocm, "lib", "libamdhip64.so")):
            try:
                _HIP = ctypes.CDLL(name, mode=ctypes.RTLD_GLOBAL)
                break
            except OSError as e:  # pragma: no cover
                last = e
        if _HIP is None:
            raise HipError("cannot load the HIP runtime: %s" % last)
        _HIP.hipGetErrorString.restype = ctypes.c_char_p
    return _HIP


def check(err, what=""):
    if err != 0:
        msg = lib().hipGetErrorString(ctypes.c_int(err))
        raise HipError("%s: hip error %d (%s)" % (what, err, msg.decode() if msg else "?"))


def device_count() -> int:
    n = ctypes.c_int(0)
    if lib().hipGetDeviceCount(ctypes.byref(n)) != 0:
        return 0
    return n.value


def set_device(i: int):
    check(lib().hipSetDevice(ctypes.c_int(i)), "hipSetDevice")


def malloc(nbytes: int) -> int:
    p = ctypes.c_void_p()
    check(lib().hipMalloc(ctypes.byref(p), ctypes.c_size_t(max(int(nbytes), 1))), "hipMalloc(%d)" % nbytes)
    return p.value


def free(ptr: int):
    check(lib().hipFree(ctypes.c_void_p(ptr)), "hipFree")


def malloc_managed(nbytes: int) -> int:
    """Managed (unified) memory, attached globally."""
    p = ctypes.c_void_p()
    check(lib().hipMallocManaged(ctypes.byref(p), ctypes.c_size_t(nbytes), ctypes.c_uint(1)), "hipMallocManaged")
    return p.value


def host_malloc(nbytes: int) -> int:
    p = ctypes.c_void_p()
    check(lib().hipHostMalloc(ctypes.byref(p), ctypes.c_size_t(nbytes), ctypes.c_uint(0)), "hipHostMalloc")
    return p.value


def host_get_device_pointer(host_ptr: int) -> int:
    """Device view of memory from host_malloc."""
    p = ctypes.c_void_p()
    check(lib().hipHostGetDevicePointer(ctypes.byref(p), ctypes.c_void_p(host_ptr), ctypes.c_uint(0)),
          "hipHostGetDevicePointer")
    return p.value


def host_free(ptr: int):
    check(lib().hipHostFree(ctypes.c_void_p(ptr)), "hipHostFree")


def memcpy_htod(dptr: int, arr: np.ndarray):
    arr = np.ascontiguousarray(arr)
    check(lib().hipMemcpy(ctypes.c_void_p(dptr), ctypes.c_void_p(arr.ctypes.data), ctypes.c_size_t(arr.nbytes),
                          ctypes.c_int(hipMemcpyHostToDevice)), "hipMemcpy H2D")


def memcpy_dtoh(arr: np.ndarray, dptr: int):
    assert arr.flags["C_CONTIGUOUS"]
    check(lib().hipMemcpy(ctypes.c_void_p(arr.ctypes.data), ctypes.c_void_p(dptr), ctypes.c_size_t(arr.nbytes),
                          ctypes.c_int(hipMemcpyDeviceToHost)), "hipMemcpy D2H")


def memcpy_raw(dst: int, src: int, nbytes: int, kind: int, stream=None):
    """hipMemcpy between two addresses; with `stream`, hipMemcpyAsync on it."""
    if stream is None:
        check(lib().hipMemcpy(ctypes.c_void_p(dst), ctypes.c_void_p(src), ctypes.c_size_t(nbytes), ctypes.c_int(kind)),
              "hipMemcpy")
    else:
        check(lib().hipMemcpyAsync(ctypes.c_void_p(dst), ctypes.c_void_p(src), ctypes.c_size_t(nbytes), ctypes.c_int(kind),
                                   ctypes.c_void_p(stream)), "hipMemcpyAsync")


def memcpy_dtod(dst: int, src: int, nbytes: int):
    check(lib().hipMemcpy(ctypes.c_void_p(dst), ctypes.c_void_p(src), ctypes.c_size_t(nbytes),
                          ctypes.c_int(hipMemcpyDeviceToDevice)), "hipMemcpy D2D")


def memset(dptr: int, value: int, nbytes: int):
    """hipMemset + device synchronize: the fill runs on the null stream and is asynchronous to the
    host, so without the wait it races with work on non-blocking streams."""
    check(lib().hipMemset(ctypes.c_void_p(dptr), ctypes.c_int(value), ctypes.c_size_t(nbytes)), "hipMemset")
    device_synchronize()


def device_synchronize():
    check(lib().hipDeviceSynchronize(), "hipDeviceSynchronize")


def stream_create(nonblocking: bool = True) -> int:
    s = ctypes.c_void_p()
    check(lib().hipStreamCreateWithFlags(ctypes.byref(s), ctypes.c_uint(hipStreamNonBlocking if nonblocking else 0)),
          "hipStreamCreateWithFlags")
    return s.value


def stream_destroy(s: int):
    check(lib().hipStreamDestroy(ctypes.c_void_p(s)), "hipStreamDestroy")


def stream_synchronize(s):
    check(lib().hipStreamSynchronize(ctypes.c_void_p(s)), "hipStreamSynchronize")


def event_create() -> int:
    e = ctypes.c_void_p()
    check(lib().hipEventCreate(ctypes.byref(e)), "hipEventCreate")
    return e.value


def event_destroy(e: int):
    check(lib().hipEventDestroy(ctypes.c_void_p(e)), "hipEventDestroy")


def event_record(e: int, stream):
    check(lib().hipEventRecord(ctypes.c_void_p(e), ctypes.c_void_p(stream)), "hipEventRecord")


def event_synchronize(e: int):
    check(lib().hipEventSynchronize(ctypes.c_void_p(e)), "hipEventSynchronize")


def event_elapsed_ms(start: int, stop: int) -> float:
    ms = ctypes.c_float(0)
    check(lib().hipEventElapsedTime(ctypes.byref(ms), ctypes.c_void_p(start), ctypes.c_void_p(stop)),
          "hipEventElapsedTime")
    return ms.value


def device_name(i: int = 0) -> str:
    buf = ctypes.create_string_buffer(256)
    check(lib().hipDeviceGetName(buf, ctypes.c_int(256), ctypes.c_int(i)), "hipDeviceGetName")
    return buf.value.decode() or "device %d" % i     # some boxes report an empty marketing name


def device_attribute(attr: int, dev: int = 0) -> int:
    v = ctypes.c_int(0)
    check(lib().hipDeviceGetAttribute(ctypes.byref(v), ctypes.c_int(attr), ctypes.c_int(dev)), "hipDeviceGetAttribute")
    return v.value


def mem_get_info():
    free_b, total_b = ctypes.c_size_t(0), ctypes.c_size_t(0)
    check(lib().hipMemGetInfo(ctypes.byref(free_b), ctypes.byref(total_b)), "hipMemGetInfo")
    return free_b.value, total_b.value


class DeviceBuffer:
    """A hipMalloc'ed region; freed on close() / garbage collection."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        self.ptr = malloc(self.nbytes)

    def upload(self, arr: np.ndarray, offset: int = 0):
        assert offset + arr.nbytes <= self.nbytes
        memcpy_htod(self.ptr + offset, arr)

    def download(self, dtype, count: int, offset: int = 0) -> np.ndarray:
        out = np.empty(count, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        if out.nbytes:
            memcpy_dtoh(out, self.ptr + offset)
        return out

    def close(self):
        if self.ptr:
            free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# ---- stream capture / graphs (for callers that record the component's launches into their own graph) ----

def stream_begin_capture(s: int, mode: int = 0):
    check(lib().hipStreamBeginCapture(ctypes.c_void_p(s), ctypes.c_int(mode)), "hipStreamBeginCapture")


def stream_end_capture(s: int) -> int:
    g = ctypes.c_void_p()
    check(lib().hipStreamEndCapture(ctypes.c_void_p(s), ctypes.byref(g)), "hipStreamEndCapture")
    return g.value


def graph_instantiate(graph: int) -> int:
    e = ctypes.c_void_p()
    check(lib().hipGraphInstantiate(ctypes.byref(e), ctypes.c_void_p(graph), None, None, ctypes.c_size_t(0)),
          "hipGraphInstantiate")
    return e.value


def graph_launch(graph_exec: int, s: int):
    check(lib().hipGraphLaunch(ctypes.c_void_p(graph_exec), ctypes.c_void_p(s)), "hipGraphLaunch")


def graph_destroy(graph: int, graph_exec: int = 0):
    if graph_exec:
        check(lib().hipGraphExecDestroy(ctypes.c_void_p(graph_exec)), "hipGraphExecDestroy")
    check(lib().hipGraphDestroy(ctypes.c_void_p(graph)), "hipGraphDestroy")
