"""ctypes mirror of the mem-component boundary (include/xccl_rocm_mem_component.h,
include/xccl_rocm_kernels.h).

Function names, argument order and status codes are those of the reference
dispatcher (src/utils/mem_component.h:52-95); every function returns the
``xccl_status_t`` as ``Status`` and raises nothing for an XCCL error, so tests
can assert on codes the way the reference's callers would.  Loading fails
loudly when the libraries are not built -- there is no Python or CPU stand-in
for the arithmetic.
"""
import ctypes
import os

from .build import LIB_DIR, built
from .types import MemType, Status, StreamType

_c = ctypes
_vp, _sz, _int = _c.c_void_p, _c.c_size_t, _c.c_int


class XcclStream(_c.Structure):
    """xccl_stream_t: ``stream`` points AT a hipStream_t."""
    _fields_ = [("type", _int), ("stream", _vp)]


class McBuf(_c.Structure):
    _fields_ = [("buf", _vp), ("size", _sz), ("used", _int)]


_ST = _int  # xccl_status_t


class MemComponentVtable(_c.Structure):
    """xccl_mem_component_t (reference src/utils/mem_component.h:28-49)."""
    _fields_ = [
        ("open", _c.CFUNCTYPE(_ST)),
        ("mem_alloc", _c.CFUNCTYPE(_ST, _c.POINTER(_vp), _sz)),
        ("mem_free", _c.CFUNCTYPE(_ST, _vp)),
        ("mem_type", _c.CFUNCTYPE(_ST, _vp, _c.POINTER(_int))),
        ("reduce", _c.CFUNCTYPE(_ST, _vp, _vp, _vp, _sz, _int, _int)),
        ("reduce_multi", _c.CFUNCTYPE(_ST, _vp, _vp, _vp, _sz, _sz, _sz, _int, _int)),
        ("memcpy_async", _c.CFUNCTYPE(_ST, _vp, _vp, _sz, _c.POINTER(XcclStream))),
        ("event_record", _c.CFUNCTYPE(_ST, _c.POINTER(XcclStream), _c.POINTER(_vp))),
        ("event_query", _c.CFUNCTYPE(_ST, _vp)),
        ("event_free", _c.CFUNCTYPE(_ST, _vp)),
        ("start_stream_activity", _c.CFUNCTYPE(_ST, _c.POINTER(XcclStream), _c.POINTER(_vp))),
        ("finish_stream_activity", _c.CFUNCTYPE(_ST, _vp)),
        ("close", _c.CFUNCTYPE(None)),
        ("dlhandle", _vp),
        ("cache", McBuf),
    ]


class RocmMemComponent(_c.Structure):
    """xccl_rocm_mem_component_t: the vtable plus the stream-ordered extension."""
    _fields_ = [
        ("super", MemComponentVtable),
        ("ext_version", _c.c_uint32),
        ("reduce_nb", _c.CFUNCTYPE(_ST, _vp, _vp, _vp, _sz, _int, _int, _c.POINTER(XcclStream), _c.POINTER(_vp))),
        ("reduce_multi_nb", _c.CFUNCTYPE(_ST, _vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _c.POINTER(XcclStream),
                                         _c.POINTER(_vp))),
        ("event_wait", _c.CFUNCTYPE(_ST, _vp)),
        ("get_stream", _c.CFUNCTYPE(_ST, _c.POINTER(_vp))),
    ]


COMPONENT_SO = os.path.join(LIB_DIR, "xccl_rocm_mem_component.so")
DISPATCH_SO = os.path.join(LIB_DIR, "libxccl_mc.so")
REPLAY_SO = os.path.join(LIB_DIR, "libxccl_ucx_replay.so")
BENCHKIT_SO = os.path.join(LIB_DIR, "libxccl_rocm_benchkit.so")

_component_lib = None
_dispatch_lib = None
_datagen_lib = None


def _need_built():
    if not built():
        raise RuntimeError(
            "xccl_amd: native libraries missing under %s -- run `python -m xccl_amd.build` "
            "(there is no CPU fallback)" % LIB_DIR)


def component_lib():
    """xccl_rocm_mem_component.so, loaded directly (kernel ABI + exported vtable)."""
    global _component_lib
    if _component_lib is None:
        _need_built()
        lib = _c.CDLL(COMPONENT_SO, mode=_c.RTLD_GLOBAL)
        lib.xccl_rocm_reduce_supported.argtypes = [_int, _int]
        lib.xccl_rocm_reduce_impl.argtypes = [_vp, _vp, _vp, _sz, _int, _int, _vp]
        lib.xccl_rocm_reduce_multi_impl.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _vp]
        lib.xccl_rocm_reduce_multi_graph.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _vp]
        lib.xccl_rocm_graph_cache_destroy.argtypes = []
        lib.xccl_rocm_graph_cache_destroy.restype = None
        lib.xccl_rocm_set_launch_shape.argtypes = [_int, _int]
        lib.xccl_rocm_set_launch_shape.restype = None
        lib.xccl_rocm_set_burst_max_grid.argtypes = [_int]
        lib.xccl_rocm_set_burst_max_grid.restype = None
        lib.xccl_rocm_direct_launch_count.argtypes = []
        lib.xccl_rocm_direct_launch_count.restype = _c.c_uint64
        lib.xccl_rocm_set_direct_queue.argtypes = [_int]
        lib.xccl_rocm_set_direct_queue.restype = None
        lib.xccl_rocm_reduce_multi_route.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _int,
                                                     _c.POINTER(_c.c_uint), _c.POINTER(_c.c_uint), _c.POINTER(_int),
                                                     _c.POINTER(_int)]
        lib.xccl_rocm_set_counted_grid.argtypes = [_int, _int]
        lib.xccl_rocm_set_counted_grid.restype = None
        lib.xccl_rocm_set_direct_tail.argtypes = [_int]
        lib.xccl_rocm_set_direct_tail.restype = None
        lib.xccl_rocm_set_direct_confirm.argtypes = [_int]
        lib.xccl_rocm_set_direct_confirm.restype = None
        lib.xccl_rocm_set_direct_options.argtypes = [_int] * 5
        lib.xccl_rocm_set_direct_options.restype = None
        lib.xccl_rocm_set_slot_max_grid.argtypes = [_int]
        lib.xccl_rocm_set_slot_max_grid.restype = None
        lib.xccl_rocm_reduce_multi_slots.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _vp, _vp, _vp,
                                                     _c.c_uint32, _c.c_uint32, _c.POINTER(_int)]
        _u32p = _c.POINTER(_c.c_uint32)
        lib.xccl_rocm_reduce_multi_flagged.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _vp, _vp, _vp,
                                                       _c.c_uint32, _c.POINTER(_int)]
        lib.xccl_rocm_reduce_multi_flagged_static.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _vp, _vp,
                                                              _c.c_uint32]
        lib.xccl_rocm_reduce_multi_graph_flagged.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _vp, _vp, _vp,
                                                             _c.c_uint32, _c.POINTER(_int), _c.POINTER(_c.c_uint64)]
        lib.xccl_rocm_reduce_multi_plan.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int,
                                                    _c.POINTER(_c.c_uint), _c.POINTER(_c.c_uint), _c.c_char_p, _sz]
        lib.xccl_rocm_stream_gate.argtypes = [_vp, _c.c_uint64, _vp]
        _component_lib = lib
    return _component_lib


def component() -> RocmMemComponent:
    """The exported object `xccl_rocm_mem_component`."""
    return RocmMemComponent.in_dll(component_lib(), "xccl_rocm_mem_component")


def bind_dispatcher(path, mode=_c.DEFAULT_MODE):
    """Loads a library that exports the xccl_mem_component_* dispatcher API
    (reference src/utils/mem_component.h:52-95) and sets the argument types of
    the entries it has: libxccl_mc.so, or a build of the reference's own
    src/utils/mem_component.c (the *_nb entries exist there only with
    integration/xccl-rocm.patch applied; event_wait / get only in libxccl_mc.so)."""
    lib = _c.CDLL(path, mode=mode)
    sigs = {
        "xccl_mem_component_init": [_c.c_char_p],
        "xccl_mem_component_alloc": [_c.POINTER(_vp), _sz, _int],
        "xccl_mem_component_free": [_vp, _int],
        "xccl_mem_component_type": [_vp, _c.POINTER(_int)],
        "xccl_mem_component_reduce": [_vp, _vp, _vp, _sz, _int, _int, _int],
        "xccl_mem_component_reduce_multi": [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _int],
        "xccl_mem_component_reduce_nb": [_vp, _vp, _vp, _sz, _int, _int, _int, _c.POINTER(XcclStream),
                                         _c.POINTER(_vp)],
        "xccl_mem_component_reduce_multi_nb": [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _int,
                                               _c.POINTER(XcclStream), _c.POINTER(_vp)],
        "xccl_mem_component_memcpy_async": [_vp, _vp, _sz, _c.POINTER(XcclStream)],
        "xccl_mem_component_start_acitivity": [_c.POINTER(XcclStream), _c.POINTER(_vp)],
        "xccl_mem_component_finish_acitivity": [_vp],
        "xccl_mc_event_record": [_c.POINTER(XcclStream), _c.POINTER(_vp)],
        "xccl_mc_event_query": [_vp],
        "xccl_mc_event_free": [_vp],
        "xccl_mc_event_wait": [_vp],
        "xccl_mem_component_free_cache": [],
        "xccl_mem_component_finalize": [],
        "xccl_mem_component_get": [_int],
    }
    for name, argtypes in sigs.items():
        fn = getattr(lib, name, None)
        if fn is None:
            continue
        fn.argtypes = argtypes
        fn.restype = _ST
    for name in ("xccl_mem_component_free_cache", "xccl_mem_component_finalize"):
        getattr(lib, name).restype = None
    if hasattr(lib, "xccl_mem_component_get"):
        lib.xccl_mem_component_get.restype = _c.POINTER(MemComponentVtable)
    return lib


def dispatch_lib():
    global _dispatch_lib
    if _dispatch_lib is None:
        _need_built()
        _dispatch_lib = bind_dispatcher(DISPATCH_SO)
    return _dispatch_lib


def benchkit_lib():
    global _datagen_lib
    if _datagen_lib is None:
        _need_built()
        lib = _c.CDLL(BENCHKIT_SO)
        lib.xccl_rocm_datagen_fill.argtypes = [_vp, _sz, _int, _c.c_uint64, _c.c_uint64, _int, _vp]
        lib.xccl_rocm_bench_copy.argtypes = [_vp, _vp, _sz, _vp]
        lib.xccl_rocm_bench_latency.argtypes = [_vp, _vp, _int, _vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _sz, _vp]
        lib.xccl_rocm_bench_kernel_times.argtypes = [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _sz, _vp, _vp]
        lib.xccl_rocm_bench_region_time.argtypes = [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _sz, _vp, _vp, _vp]
        lib.xccl_rocm_bench_region_time_rot.argtypes = [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _int, _int, _sz,
                                                        _vp, _vp, _vp]
        lib.xccl_rocm_bench_latency_mt.argtypes = [_vp, _int, _sz, _vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _sz, _vp]
        lib.xccl_rocm_bench_memcpy.argtypes = [_vp, _vp, _vp, _vp, _sz, _sz, _vp]
        lib.xccl_rocm_bench_mem_type.argtypes = [_vp, _vp, _sz, _vp, _vp]
        lib.xccl_rocm_bench_alloc_free.argtypes = [_vp, _sz, _sz, _vp]
        lib.xccl_rocm_bench_graph_parts.argtypes = [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _sz, _vp]
        lib.xccl_rocm_bench_read.argtypes = [_vp, _sz, _c.c_uint, _sz, _c.c_uint, _vp, _vp]
        _datagen_lib = lib
    return _datagen_lib


def _st(code) -> Status:
    try:
        return Status(code)
    except ValueError:
        return code


class Stream:
    """Owns a hipStream_t and the xccl_stream_t that points at it."""

    def __init__(self, hip_stream, stype=StreamType.ROCM):
        self._handle = _vp(hip_stream)
        self.xccl = XcclStream(int(stype), _c.cast(_c.pointer(self._handle), _vp))

    @property
    def hip_stream(self):
        return self._handle.value

    def ref(self):
        return _c.byref(self.xccl)


# ---- dispatcher mirror (reference src/utils/mem_component.c) ----------------

def xccl_mem_component_init(path: str = LIB_DIR) -> Status:
    return _st(dispatch_lib().xccl_mem_component_init(path.encode()))


def xccl_mem_component_alloc(nbytes: int, mem_type):
    p = _vp()
    st = dispatch_lib().xccl_mem_component_alloc(_c.byref(p), nbytes, int(mem_type))
    return _st(st), p.value


def xccl_mem_component_free(ptr, mem_type) -> Status:
    return _st(dispatch_lib().xccl_mem_component_free(ptr, int(mem_type)))


def xccl_mem_component_type(ptr):
    mt = _int(-1)
    st = dispatch_lib().xccl_mem_component_type(ptr, _c.byref(mt))
    return _st(st), MemType(mt.value)


def xccl_mem_component_reduce(sbuf1, sbuf2, target, count, dtype, op, mem_type) -> Status:
    return _st(dispatch_lib().xccl_mem_component_reduce(sbuf1, sbuf2, target, count, int(dtype), int(op),
                                                        int(mem_type)))


def xccl_mem_component_reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, mem_type) -> Status:
    return _st(dispatch_lib().xccl_mem_component_reduce_multi(sbuf1, sbuf2, rbuf, count, size, stride, int(dtype),
                                                              int(op), int(mem_type)))


def xccl_mem_component_reduce_nb(sbuf1, sbuf2, target, count, dtype, op, mem_type, stream=None, want_event=True):
    ev = _vp()
    st = dispatch_lib().xccl_mem_component_reduce_nb(sbuf1, sbuf2, target, count, int(dtype), int(op), int(mem_type),
                                                     stream.ref() if stream else None,
                                                     _c.byref(ev) if want_event else None)
    return _st(st), ev.value


def xccl_mem_component_reduce_multi_nb(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, mem_type, stream=None,
                                       want_event=True):
    ev = _vp()
    st = dispatch_lib().xccl_mem_component_reduce_multi_nb(sbuf1, sbuf2, rbuf, count, size, stride, int(dtype),
                                                           int(op), int(mem_type),
                                                           stream.ref() if stream else None,
                                                           _c.byref(ev) if want_event else None)
    return _st(st), ev.value


def xccl_mem_component_memcpy_async(sbuf, dbuf, size, stream: Stream) -> Status:
    return _st(dispatch_lib().xccl_mem_component_memcpy_async(sbuf, dbuf, size, stream.ref()))


def xccl_mem_component_start_acitivity(stream: Stream):
    req = _vp()
    st = dispatch_lib().xccl_mem_component_start_acitivity(stream.ref(), _c.byref(req))
    return _st(st), req.value


def xccl_mem_component_finish_acitivity(req) -> Status:
    return _st(dispatch_lib().xccl_mem_component_finish_acitivity(req))


def xccl_mc_event_record(stream: Stream):
    ev = _vp()
    st = dispatch_lib().xccl_mc_event_record(stream.ref(), _c.byref(ev))
    return _st(st), ev.value


def xccl_mc_event_query(ev) -> Status:
    return _st(dispatch_lib().xccl_mc_event_query(ev))


def xccl_mc_event_free(ev) -> Status:
    return _st(dispatch_lib().xccl_mc_event_free(ev))


def xccl_mc_event_wait(ev) -> Status:
    return _st(dispatch_lib().xccl_mc_event_wait(ev))


def xccl_mem_component_free_cache():
    dispatch_lib().xccl_mem_component_free_cache()


def xccl_mem_component_finalize():
    dispatch_lib().xccl_mem_component_finalize()


def component_stream():
    """hipStream_t (int) the component's synchronous entries launch on."""
    s = _vp()
    st = component().get_stream(_c.byref(s))
    if st != 0:
        raise RuntimeError("get_stream failed: %s" % _st(st))
    return s.value


def datagen_fill(dptr, count, dtype, seed, vec, sparse=False, hip_stream=None) -> Status:
    return _st(benchkit_lib().xccl_rocm_datagen_fill(dptr, count, int(dtype), seed, vec, int(bool(sparse)),
                                                    hip_stream))


def bench_copy(dst, src, nbytes, hip_stream=None) -> Status:
    return _st(benchkit_lib().xccl_rocm_bench_copy(dst, src, nbytes, hip_stream))


LATENCY_MODES = {"sync": 0, "event": 1, "graph": 2, "stream": 3, "issue": 4}


def bench_latency(mode: str, sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, iters: int):
    """Per-call host-observed durations in ns (numpy uint64) of `iters`
    back-to-back reduce_multi calls; see csrc/bench_loops.c for the modes."""
    import numpy as np
    out = np.zeros(iters, dtype=np.uint64)
    comp = _c.addressof(component())
    graph_fn = _c.cast(component_lib().xccl_rocm_reduce_multi_graph, _vp)
    st = benchkit_lib().xccl_rocm_bench_latency(comp, graph_fn, LATENCY_MODES[mode], sbuf1, sbuf2, rbuf, count, size,
                                                stride, int(dtype), int(op), iters, out.ctypes.data)
    return _st(st), out


def bench_kernel_times(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, iters: int):
    """Device-side duration in ms (numpy float32) of each of `iters` launches,
    from HIP event pairs recorded on the component stream around each launch."""
    import numpy as np
    from . import hip
    evs = (_vp * (2 * iters))(*[hip.event_create() for _ in range(2 * iters)])
    out = np.zeros(iters, dtype=np.float32)
    st = benchkit_lib().xccl_rocm_bench_kernel_times(_c.addressof(component()), sbuf1, sbuf2, rbuf, count, size, stride,
                                                     int(dtype), int(op), iters, evs, out.ctypes.data)
    for e in evs:
        hip.event_destroy(e)
    return _st(st), out


def reduce_multi_plan(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op):
    """What a launch with these arguments would be: mangled kernel name, grid and block size."""
    grid, block, name = _c.c_uint(0), _c.c_uint(0), _c.create_string_buffer(256)
    st = component_lib().xccl_rocm_reduce_multi_plan(sbuf1, sbuf2, rbuf, count, size, stride, int(dtype), int(op),
                                                     _c.byref(grid), _c.byref(block), name, 256)
    if _st(st) != Status.OK:
        raise RuntimeError("xccl_rocm_reduce_multi_plan: %s" % _st(st))
    return {"kernel": name.value.decode(), "grid": grid.value, "block": block.value}


ROUTES = ("stream", "slots", "counted", "tail", "signal")     # XCCL_ROCM_ROUTE_*


def reduce_multi_route(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, own_queue=False):
    """What a launch that reports its own completion would be, on a HIP stream or on the component's own
    queue: grid, LDS bytes asked for to bound residency, burst kernel or not, completion route."""
    grid, lds, burst, route = _c.c_uint(0), _c.c_uint(0), _int(0), _int(0)
    st = component_lib().xccl_rocm_reduce_multi_route(sbuf1, sbuf2, rbuf, count, size, stride, int(dtype), int(op),
                                                      int(bool(own_queue)), _c.byref(grid), _c.byref(lds),
                                                      _c.byref(burst), _c.byref(route))
    if _st(st) != Status.OK:
        raise RuntimeError("xccl_rocm_reduce_multi_route: %s" % _st(st))
    return {"grid": grid.value, "lds_bytes": lds.value, "burst": bool(burst.value), "route": ROUTES[route.value]}


def bench_region_time_rot(sbuf1, sbuf2, rbuf, rot_count, rot_pitch, count, size, stride, dtype, op, iters: int):
    """bench_region_time with the destination cycling through `rot_count` vectors `rot_pitch` bytes apart."""
    from . import hip
    e0, e1 = hip.event_create(), hip.event_create()
    ms = _c.c_float(0)
    st = benchkit_lib().xccl_rocm_bench_region_time_rot(_c.addressof(component()), sbuf1, sbuf2, rbuf, rot_count,
                                                        rot_pitch, count, size, stride, int(dtype), int(op), iters,
                                                        e0, e1, _c.byref(ms))
    hip.event_destroy(e0)
    hip.event_destroy(e1)
    return _st(st), ms.value


def bench_region_time(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, iters: int):
    """Device time in ms of `iters` back-to-back launches on the component stream,
    from ONE pair of HIP events around them all."""
    from . import hip
    e0, e1 = hip.event_create(), hip.event_create()
    ms = _c.c_float(0)
    st = benchkit_lib().xccl_rocm_bench_region_time(_c.addressof(component()), sbuf1, sbuf2, rbuf, count, size, stride,
                                                    int(dtype), int(op), iters, e0, e1, _c.byref(ms))
    hip.event_destroy(e0)
    hip.event_destroy(e1)
    return _st(st), ms.value


def bench_graph_parts(sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, iters: int):
    """Host time in ns of the steps of a one-node graph launch with a completion word, `iters` rounds x
    (planning, lock + slot search, patching, hipGraphLaunch, completion seen, whole round)."""
    import numpy as np
    out = np.zeros((iters, 6), dtype=np.uint64)
    fn = _c.cast(component_lib().xccl_rocm_reduce_multi_graph_flagged, _vp)
    st = benchkit_lib().xccl_rocm_bench_graph_parts(_c.addressof(component()), fn, sbuf1, sbuf2, rbuf, count, size,
                                                    stride, int(dtype), int(op), iters, out.ctypes.data)
    return _st(st), out


def bench_read(src, stride, nsrc, nbytes, lds_bytes=0, hip_stream=None) -> Status:
    """Read-only kernel with the reduction's access pattern (nothing is written)."""
    return _st(benchkit_lib().xccl_rocm_bench_read(src, stride, nsrc, nbytes, lds_bytes, None, hip_stream))


def bench_latency_mt(threads: int, thread_pitch: int, sbuf1, sbuf2, rbuf, count, size, stride, dtype, op, iters: int):
    """Per-call durations in ns, shape (threads, iters), of blocking reduce_multi calls
    issued by `threads` host threads at once, thread t on operands t * thread_pitch further on."""
    import numpy as np
    out = np.zeros((threads, iters), dtype=np.uint64)
    st = benchkit_lib().xccl_rocm_bench_latency_mt(_c.addressof(component()), threads, thread_pitch, sbuf1, sbuf2, rbuf,
                                                   count, size, stride, int(dtype), int(op), iters, out.ctypes.data)
    return _st(st), out


def bench_memcpy(stream: Stream, src, dst, nbytes: int, iters: int):
    """Durations in ns of `iters` rounds of memcpy_async + event_record + event_query polling."""
    import numpy as np
    out = np.zeros(iters, dtype=np.uint64)
    st = benchkit_lib().xccl_rocm_bench_memcpy(_c.addressof(component()), stream.ref(), src, dst, nbytes, iters,
                                               out.ctypes.data)
    return _st(st), out


def bench_mem_type(ptr, iters: int):
    """Durations in ns (numpy uint64) of `iters` mem_type probes of `ptr` through the
    component's vtable, and the memory type the last probe reported (None: not recognised)."""
    import numpy as np
    out = np.zeros(iters, dtype=np.uint64)
    mt = _c.c_int(0)
    st = benchkit_lib().xccl_rocm_bench_mem_type(_c.addressof(component()), ptr, iters, out.ctypes.data, _c.byref(mt))
    return _st(st), out, (None if mt.value == int(MemType.LAST) else MemType(mt.value))


def bench_alloc_free(nbytes: int, iters: int):
    """Durations in ns (numpy uint64) of `iters` mem_alloc(nbytes) + mem_free pairs
    through the component's vtable."""
    import numpy as np
    out = np.zeros(iters, dtype=np.uint64)
    st = benchkit_lib().xccl_rocm_bench_alloc_free(_c.addressof(component()), nbytes, iters, out.ctypes.data)
    return _st(st), out


class MemPoolStats(_c.Structure):
    """include/xccl_rocm_mem_pool.h: xccl_rocm_mem_pool_stats_t"""
    _fields_ = [("hits", _c.c_uint64), ("misses", _c.c_uint64), ("backing_frees", _c.c_uint64),
                ("cached_bytes", _c.c_size_t), ("live_blocks", _c.c_size_t), ("free_blocks", _c.c_size_t)]


def mem_pool_set_limit(limit_bytes: int) -> None:
    fn = component_lib().xccl_rocm_mem_pool_set_limit
    fn.argtypes, fn.restype = [_sz], None
    fn(limit_bytes)


def mem_pool_stats() -> MemPoolStats:
    fn = component_lib().xccl_rocm_mem_pool_get_stats
    fn.argtypes, fn.restype = [_c.POINTER(MemPoolStats)], None
    out = MemPoolStats()
    fn(_c.byref(out))
    return out


# ---- UCX team-library call sites over a loopback transport (include/xccl_rocm_ucx_replay.h) ----

class ReplayParams(_c.Structure):
    _fields_ = [("alg", _int), ("reduce_mode", _int), ("team_size", _int), ("radix", _int), ("root", _int),
                ("count", _sz), ("dtype", _int), ("op", _int), ("src", _c.POINTER(_vp)), ("dst", _c.POINTER(_vp))]


class ReplayStats(_c.Structure):
    _fields_ = [(n, _c.c_uint64) for n in (
        "reduce_calls", "reduce_multi_calls", "max_multi_vectors", "inplace_sbuf1", "inplace_sbuf2", "messages",
        "bytes_moved", "progress_calls", "reduce_inflight_returns", "scratch_allocs")]

    def as_dict(self):
        return {n: int(getattr(self, n)) for n, _ in self._fields_}


REPLAY_ALGS = {"allreduce_knomial": 0, "allreduce_sra": 1, "reduce_knomial": 2, "reduce_linear": 3}
_replay_lib = None


def replay_lib():
    global _replay_lib
    if _replay_lib is None:
        _need_built()
        dispatch_lib()
        lib = _c.CDLL(REPLAY_SO)
        lib.xccl_replay_run.argtypes = [_c.POINTER(ReplayParams), _c.POINTER(ReplayStats), _c.c_uint64]
        lib.xccl_replay_knomial_geometry.argtypes = [_int, _int, _int, _c.POINTER(_int), _c.POINTER(_int),
                                                     _c.POINTER(_int)]
        lib.xccl_replay_knomial_geometry.restype = None
        lib.xccl_replay_sra_segment.argtypes = [_sz, _int, _int, _int, _c.POINTER(_sz), _c.POINTER(_sz)]
        lib.xccl_replay_sra_segment.restype = None
        _replay_lib = lib
    return _replay_lib


def replay_run(alg: str, src_ptrs, dst_ptrs, count, dtype, op, radix=4, root=0, stream_ordered=True, max_sweeps=0):
    """One collective over len(src_ptrs) loopback ranks; returns (Status, stats dict)."""
    n = len(src_ptrs)
    src = (_vp * n)(*src_ptrs)
    dst = (_vp * n)(*dst_ptrs)
    prm = ReplayParams(REPLAY_ALGS[alg], 1 if stream_ordered else 0, n, radix, root, count, int(dtype), int(op),
                       _c.cast(src, _c.POINTER(_vp)), _c.cast(dst, _c.POINTER(_vp)))
    stats = ReplayStats()
    st = replay_lib().xccl_replay_run(_c.byref(prm), _c.byref(stats), max_sweeps)
    return _st(st), stats.as_dict()


def knomial_geometry(radix, rank, team_size):
    """(rounds, full_size, role) with role 0 = base, 1 = proxy, 2 = extra."""
    a, b, r = _int(0), _int(0), _int(0)
    replay_lib().xccl_replay_knomial_geometry(radix, rank, team_size, _c.byref(a), _c.byref(b), _c.byref(r))
    return a.value, b.value, r.value


def sra_segment(count, rank, radix, team_size):
    """(element offset, length) of the segment `rank` owns after the scatter-reduce."""
    o, n = _sz(0), _sz(0)
    replay_lib().xccl_replay_sra_segment(count, rank, radix, team_size, _c.byref(o), _c.byref(n))
    return o.value, n.value
