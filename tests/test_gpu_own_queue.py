"""The component's own dispatch queues beyond the basics: what a launch there
may assume about inputs that somebody other than a kernel has just rewritten,
the knobs that decide which calls go there and how they complete, and every
launch-shape variable of the environment showing in the route a call takes."""
import ctypes
import json
import os
import subprocess
import sys
import time

import numpy as np
import pytest

from gpu_util import Case, assert_same
from xccl_amd import hip
from xccl_amd.types import Dt, MemType, Op, Status

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("acquire", ["agent", "system"])
def test_sources_rewritten_in_place_between_own_queue_calls(rocm, acquire):
    """Between two rounds of a collective the scratch a reduction reads is
    rewritten at the SAME addresses by a writer that is no kernel of the
    component's queue (reference allreduce_knomial.c:104-135: receives land in
    scratch, then the reduction runs).  Here: a blocking reduction on the own
    queue; one source vector overwritten in place through a copy from pageable
    host memory, from pinned host memory (copy engine), an asynchronous copy on
    another stream, or a device-to-device copy; the reduction again on the same
    addresses; compared with numpy every round.  Launches carry an agent-scope
    acquire fence by default; the system-scope setting is run as well.  Sizes
    from cache-resident (1 KiB) to 2 MiB per vector, 2 / 4 / 8 sources, 200+
    rounds per setting; stops at the first stale element."""
    lib = rocm.component_lib()
    lib.xccl_rocm_set_direct_options(1 if acquire == "system" else 0, -1, -1, -1, -1)
    rng = np.random.default_rng(7)
    maxb = 2 << 20
    pinned = hip.host_malloc(maxb)
    pin = np.ctypeslib.as_array(ctypes.cast(pinned, ctypes.POINTER(ctypes.c_uint8)), shape=(maxb,))
    other = hip.stream_create()
    stage = hip.DeviceBuffer(maxb)
    rounds = 0
    try:
        # whichever way the first call goes: earlier tests may have left launches on the stream nobody waited for
        warm = hip.DeviceBuffer(4096)
        assert rocm.xccl_mem_component_reduce_multi(warm.ptr, warm.ptr + 1024, warm.ptr + 2048, 1, 256, 1024, Dt.INT32,
                                                    Op.SUM, MemType.ROCM) == Status.OK
        warm.close()
        for nsrc in (2, 4, 8):
            for vb in (1024, 8192, 65536, 1 << 20, 2 << 20):
                size = vb // 4
                dev = hip.DeviceBuffer((nsrc + 1) * vb)
                slab = rng.integers(-(1 << 20), 1 << 20, (nsrc, size), dtype=np.int32)
                dev.upload(slab)
                before = lib.xccl_rocm_direct_launch_count()
                n_rounds = 16
                for r in range(n_rounds):
                    st = rocm.xccl_mem_component_reduce_multi(dev.ptr, dev.ptr + vb, dev.ptr + nsrc * vb, nsrc - 1, size,
                                                              vb, Dt.INT32, Op.SUM, MemType.ROCM)
                    assert st == Status.OK
                    got = dev.download(np.int32, size, nsrc * vb)
                    want = slab.sum(axis=0, dtype=np.int32)
                    assert np.array_equal(got, want), \
                        "stale source data: acquire=%s, %d sources x %d B, round %d, %d elements differ" % (
                            acquire, nsrc, vb, r, int((got != want).sum()))
                    rounds += 1
                    j = (r // 4) % nsrc
                    new = rng.integers(-(1 << 20), 1 << 20, size, dtype=np.int32)
                    slab[j] = new
                    target = dev.ptr + j * vb
                    how = r % 4
                    if how == 0:
                        hip.memcpy_htod(target, new)
                    elif how == 1:
                        pin[:vb] = new.view(np.uint8)
                        hip.memcpy_raw(target, pinned, vb, hip.hipMemcpyHostToDevice)
                    elif how == 2:
                        pin[:vb] = new.view(np.uint8)
                        hip.memcpy_raw(target, pinned, vb, hip.hipMemcpyHostToDevice, other)
                        hip.stream_synchronize(other)
                    else:
                        stage.upload(new)
                        hip.memcpy_dtod(target, stage.ptr, vb)
                        # a device-to-device copy returns before it has run; the own queue is ordered against no
                        # stream, so the caller waits for what it depends on, as it does for a receive
                        hip.device_synchronize()
                assert lib.xccl_rocm_direct_launch_count() - before == n_rounds, "the calls did not take the own queue"
                dev.close()
        assert rounds >= 200
    finally:
        lib.xccl_rocm_set_direct_options(0, -1, -1, -1, -1)
        hip.host_free(pinned)
        hip.stream_destroy(other)
        stage.close()


def test_large_launch_on_the_own_queue_completes_through_its_signal(rocm, oracle):
    """With the second-packet completion off and the signal option on, a call
    too large to count its own workgroups stays on the own queue and completes
    through the packet's completion signal: blocking entry, reduce_multi_nb +
    event_query, and a small blocking call issued behind an unwaited large one
    (it is ordered behind it).  With both off, the same call goes to the HIP
    stream."""
    lib = rocm.component_lib()
    lib.xccl_rocm_set_direct_tail(0)
    dt, op, n2 = Dt.FLOAT32, Op.SUM, 3
    large, small = Case(dt, 3 * 1024 * 1024 + 5, n2), Case(dt, 3001, 1, alias="s1")
    try:
        large.fill_random(oracle, 71)
        large.upload()
        want = large.expect(oracle, op)[0]
        p1, p2, pr = large.ptrs()
        assert rocm.reduce_multi_route(p1, p2, pr, n2, large.size, large.stride, dt, op, own_queue=True)["route"] == "stream"
        lib.xccl_rocm_set_direct_tail(1)
        assert rocm.reduce_multi_route(p1, p2, pr, n2, large.size, large.stride, dt, op, own_queue=True)["route"] == "tail"
        lib.xccl_rocm_set_direct_tail(0)
        assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, n2, large.size, large.stride, dt, op,
                                                    MemType.ROCM) == Status.OK     # leaves the stream idle
        lib.xccl_rocm_set_direct_options(-1, -1, -1, -1, 1)
        assert rocm.reduce_multi_route(p1, p2, pr, n2, large.size, large.stride, dt, op, own_queue=True)["route"] == "signal"
        for rep in range(3):
            hip.memset(pr, 0x40 + rep, large.vbytes)
            before = lib.xccl_rocm_direct_launch_count()
            assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, n2, large.size, large.stride, dt, op,
                                                        MemType.ROCM) == Status.OK
            assert lib.xccl_rocm_direct_launch_count() - before == 1
            assert_same(large.result(), want, dt, op, "blocking, completion signal, rep %d" % rep)
        # stream-ordered, then a small in-place call of the same thread behind it
        small.fill_random(oracle, 72)
        small.upload()
        c1, c2, cr = small.ptrs()
        a = small.host[small.o1: small.o1 + small.vbytes].view(np.float32).copy()
        b = small.host[small.o2: small.o2 + small.vbytes].view(np.float32).copy()
        hip.memset(pr, 0x77, large.vbytes)
        before = lib.xccl_rocm_direct_launch_count()
        st, ev = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, n2, large.size, large.stride, dt, op, MemType.ROCM,
                                                         None)
        assert st == Status.OK and ev is not None
        assert rocm.xccl_mem_component_reduce_multi(c1, c2, cr, 1, small.size, small.stride, dt, op,
                                                    MemType.ROCM) == Status.OK
        assert lib.xccl_rocm_direct_launch_count() - before == 2
        assert rocm.xccl_mc_event_query(ev) == Status.OK        # ordered behind it, so it has completed too
        assert rocm.xccl_mc_event_free(ev) == Status.OK
        assert_same(large.result(), want, dt, op, "stream-ordered, completion signal")
        assert small.result().view(np.float32).tolist() == (a + b).tolist()
        # many events in flight, each with a signal of its own
        evs = []
        for rep in range(6):
            st, e = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, n2, large.size, large.stride, dt, op,
                                                            MemType.ROCM, None)
            assert st == Status.OK and e is not None
            evs.append(e)
        t0 = time.time()
        while rocm.xccl_mc_event_query(evs[-1]) == Status.INPROGRESS:
            assert time.time() - t0 < 20.0
        for e in evs:
            assert rocm.xccl_mc_event_query(e) == Status.OK and rocm.xccl_mc_event_free(e) == Status.OK
        assert_same(large.result(), want, dt, op, "six stream-ordered launches")
        lib.xccl_rocm_set_direct_options(-1, -1, -1, -1, 0)
        before = lib.xccl_rocm_direct_launch_count()
        assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, n2, large.size, large.stride, dt, op,
                                                    MemType.ROCM) == Status.OK
        assert lib.xccl_rocm_direct_launch_count() - before == 0
    finally:
        lib.xccl_rocm_set_direct_options(-1, -1, -1, -1, 0)
        lib.xccl_rocm_set_direct_tail(1)
        large.close()
        small.close()


@pytest.mark.parametrize("nsrc", [2, 4, 9])
def test_large_launch_on_the_own_queue_with_a_second_packet(rocm, oracle, nsrc):
    """The default for calls beyond 64 workgroups: the reduction as one packet,
    a one-lane kernel that stores the completion word as a second one behind
    it.  Blocking entry and reduce_multi_nb + event_query over sizes either
    side of every bound (64 / 65 workgroups, the burst kernel's 2048, ragged
    tiles, 12 MiB vectors), in place, and 40 events in flight at once."""
    lib = rocm.component_lib()
    dt, op, n2 = Dt.INT32, Op.SUM, nsrc - 1
    for size in (64 * 256, 64 * 256 + 1, 65 * 256 - 3, 2048 * 256, 2049 * 256 + 7, 3 * 1024 * 1024 + 5):
        c = Case(dt, size, n2, alias="s1" if size % 2 else None)
        try:
            c.fill_random(oracle, 500 + nsrc)
            c.upload()
            p1, p2, pr = c.ptrs()
            want, _ = c.expect(oracle, op)
            route = rocm.reduce_multi_route(p1, p2, pr, n2, size, c.stride, dt, op, own_queue=True)
            assert route["route"] == ("counted" if route["grid"] <= 64 else "tail"), (size, route)
            before = lib.xccl_rocm_direct_launch_count()
            assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, n2, size, c.stride, dt, op, MemType.ROCM) == Status.OK
            assert lib.xccl_rocm_direct_launch_count() - before == 1
            assert_same(c.result(), want, dt, op, "blocking, %d elements" % size)
            c.upload()
            st, ev = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, n2, size, c.stride, dt, op, MemType.ROCM, None)
            assert st == Status.OK and ev is not None
            t0 = time.time()
            while rocm.xccl_mc_event_query(ev) == Status.INPROGRESS:
                assert time.time() - t0 < 20.0
            assert rocm.xccl_mc_event_query(ev) == Status.OK and rocm.xccl_mc_event_free(ev) == Status.OK
            assert_same(c.result(), want, dt, op, "stream-ordered, %d elements" % size)
        finally:
            c.close()
    # 40 stream-ordered launches of 300 workgroups in place, none waited for until the end: 80 packets in order
    chain = Case(dt, 300 * 256, 1, alias="s1")
    try:
        chain.fill_random(oracle, 600 + nsrc)
        chain.upload()
        c1, c2, cr = chain.ptrs()
        evs = []
        for rep in range(40):
            st, e = rocm.xccl_mem_component_reduce_multi_nb(c1, c2, cr, 1, chain.size, chain.stride, dt, op, MemType.ROCM,
                                                            None)
            assert st == Status.OK and e is not None
            evs.append(e)
        t0 = time.time()
        while rocm.xccl_mc_event_query(evs[-1]) == Status.INPROGRESS:
            assert time.time() - t0 < 20.0
        for e in evs:
            assert rocm.xccl_mc_event_query(e) == Status.OK and rocm.xccl_mc_event_free(e) == Status.OK
        a = chain.host[chain.o1: chain.o1 + chain.vbytes].view(np.int32).astype(np.int64)
        b = chain.host[chain.o2: chain.o2 + chain.vbytes].view(np.int32).astype(np.int64)
        want = ((a + 40 * b) & 0xffffffff).astype(np.uint32).view(np.int32)
        assert chain.result().view(np.int32).tolist() == want.tolist()
    finally:
        chain.close()


def test_thread_slots_and_queue_sharing(rocm, oracle):
    """Four calling threads land on the component's four thread slots.  By
    default two queues serve all four slots; with sharing off the threads of
    slots 2 and 3 keep to their HIP streams; with four queues every slot has its
    own.  The launch counter tells; results are checked per thread."""
    lib = rocm.component_lib()
    iters, threads = 300, 4
    size, n2 = 256, 3
    pitch = 8192
    buf = hip.DeviceBuffer(threads * pitch)
    host = np.zeros(threads * pitch // 4, dtype=np.float32)
    for t in range(threads):
        for j in range(4):
            host[t * pitch // 4 + j * size: t * pitch // 4 + (j + 1) * size] = oracle.fill(size, Dt.FLOAT32, 300 + t, j)
    buf.upload(host)
    try:
        for queues, share, expect_all in ((2, 1, True), (2, 0, False), (4, 0, True), (1, 1, True), (2, 1, True)):
            lib.xccl_rocm_set_direct_options(-1, queues, share, -1, -1)
            hip.memset(buf.ptr + 4 * size * 4, 0, size * 4)
            before = lib.xccl_rocm_direct_launch_count()
            st, ns = rocm.bench_latency_mt(threads, pitch, buf.ptr, buf.ptr + size * 4, buf.ptr + 4 * size * 4, n2, size,
                                           size * 4, Dt.FLOAT32, Op.SUM, iters)
            assert st == Status.OK
            took = lib.xccl_rocm_direct_launch_count() - before
            if expect_all:
                assert took == threads * iters, (queues, share, took)
            else:
                assert took == threads * iters // 2, (queues, share, took)
            got = buf.download(np.float32, threads * pitch // 4, 0)
            for t in range(threads):
                base = t * pitch // 4
                want = np.empty(size, dtype=np.float32)
                src = host[base: base + 4 * size].copy()
                oracle.reduce_multi(src, src, want, n2, size, size * 4, Dt.FLOAT32, Op.SUM, off2=size * 4)
                assert got[base + 4 * size: base + 5 * size].tobytes() == want.tobytes(), (queues, share, t)
    finally:
        lib.xccl_rocm_set_direct_options(-1, 2, 1, -1, -1)
        buf.close()


KERNARG_PROBE = """
import ctypes, sys
sys.path.insert(0, %r)
import numpy as np
from xccl_amd import hip, mc
from xccl_amd.types import Dt, MemType, Op, Status
hip.set_device(0)
assert mc.xccl_mem_component_init() == Status.OK
lib = mc.component_lib()
lib.xccl_rocm_direct_kernarg_arena.restype = ctypes.c_void_p
lib.xccl_rocm_direct_kernarg_arena.argtypes = [ctypes.c_size_t]
rng = np.random.default_rng(3)
ok = True
for size in (1, 255, 4096, 100003):
    a = rng.integers(-1000, 1000, (4, size), dtype=np.int32)
    buf = hip.DeviceBuffer(5 * size * 4)
    buf.upload(a)
    before = lib.xccl_rocm_direct_launch_count()
    for rep in range(50):
        assert mc.xccl_mem_component_reduce_multi(buf.ptr, buf.ptr + size * 4, buf.ptr + 4 * size * 4, 3, size, size * 4,
                                                  Dt.INT32, Op.SUM, MemType.ROCM) == Status.OK
    ok = ok and lib.xccl_rocm_direct_launch_count() - before == 50
    ok = ok and bool((buf.download(np.int32, size, 4 * size * 4) == a.sum(axis=0, dtype=np.int32)).all())
    buf.close()
first = lib.xccl_rocm_direct_kernarg_arena(8192)
print("arena", bool(first), first == lib.xccl_rocm_direct_kernarg_arena(4096), lib.xccl_rocm_direct_kernarg_arena(1 << 20) is None, "ok", ok)
"""


def test_kernel_arguments_in_device_memory_and_in_pinned_memory():
    """Launches on the own queues read their arguments from device memory that
    the host writes through the PCIe aperture (one arena per device, the same
    memory on every request that fits, none for a larger one); with
    XCCL_MC_ROCM_DEVICE_KERNARG=0 they read them from pinned host memory.  Between
    writing such a block and the doorbell the host writes the device's
    host-data-path flush register (default), also reads it back, reads the
    block back, or does neither (XCCL_MC_ROCM_DIRECT_CONFIRM = 1, 2, 3, 0).
    Every way: 200 blocking calls on the own queue, results as numpy's."""
    for env, arena in (({}, "True True True"), ({"XCCL_MC_ROCM_DEVICE_KERNARG": "0"}, "False True True"),
                       ({"XCCL_MC_ROCM_DIRECT_CONFIRM": "0"}, "True True True"),
                       ({"XCCL_MC_ROCM_DIRECT_CONFIRM": "2"}, "True True True"),
                       ({"XCCL_MC_ROCM_DIRECT_CONFIRM": "3"}, "True True True")):
        e = dict(os.environ)
        e.pop("XCCL_MC_ROCM_DEVICE_KERNARG", None)
        e.pop("XCCL_MC_ROCM_DIRECT_CONFIRM", None)
        e.update(env)
        out = subprocess.run([sys.executable, "-c", KERNARG_PROBE % ROOT], env=e, capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stdout + out.stderr
        assert "arena %s ok True" % arena in out.stdout, (env, out.stdout + out.stderr)


ROUTE_PROBE = """
import json, sys
sys.path.insert(0, %r)
from xccl_amd import hip, mc
from xccl_amd.types import Dt, Op
hip.set_device(0)
out = {}
for name, nsrc, tiles in (("four_tiles", 4, 4), ("small_4src", 4, 1000), ("mid", 8, 4096), ("large", 8, 16384),
                          ("huge", 8, 262144)):
    size = tiles * 256
    vb = size * 4
    for own in (False, True):
        out[name + ("_own" if own else "_stream")] = mc.reduce_multi_route(0x10000000, 0x10000000 + vb, 0x10000000 + nsrc * vb,
                                                                           nsrc - 1, size, vb, Dt.FLOAT32, Op.SUM, own)
print(json.dumps(out))
"""


def _routes(env):
    e = dict(os.environ)
    for k in list(e):
        if k.startswith("XCCL_MC_ROCM_"):
            del e[k]
    e.update(env)
    out = subprocess.run([sys.executable, "-c", ROUTE_PROBE % ROOT], env=e, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    return json.loads(out.stdout.strip().splitlines()[-1])


def test_every_launch_shape_variable_changes_the_route_it_names():
    """Each XCCL_MC_ROCM_* launch-shape variable, set in the environment of a
    fresh process, changes exactly what it names in the plan of a call."""
    d = _routes({})
    assert d["four_tiles_stream"] == {"grid": 4, "lds_bytes": 0, "burst": True, "route": "slots"}
    assert d["four_tiles_own"]["route"] == "slots"
    assert d["small_4src_own"] == {"grid": 1000, "lds_bytes": 0, "burst": True, "route": "tail"}
    assert d["mid_stream"]["route"] == "tail" and d["mid_own"]["route"] == "tail" and not d["mid_own"]["burst"]
    assert d["large_stream"]["route"] == "tail" and d["large_own"]["route"] == "tail" and d["huge_own"]["route"] == "tail"
    n = _routes({"XCCL_MC_ROCM_DIRECT_TAIL": "0"})
    assert n["small_4src_own"]["route"] == "counted" and n["mid_own"]["route"] == "counted"     # up to 6144 workgroups
    assert n["large_own"]["route"] == "stream" and n["large_stream"] == d["large_stream"]
    assert d["huge_stream"] == {"grid": 262144, "lds_bytes": 10752, "burst": False, "route": "tail"}   # 15 resident per CU
    assert d["mid_stream"]["lds_bytes"] == 0           # 9 x 4 MiB: fits the memory-side cache, no residency bound

    c = _routes({"XCCL_MC_ROCM_MAX_COUNTED_GRID": "5000"})
    assert c["mid_stream"]["route"] == "counted" and c["mid_own"]["route"] == "counted" and c["large_stream"]["route"] == "tail"
    assert c["large_own"]["route"] == "tail"
    c = _routes({"XCCL_MC_ROCM_MAX_COUNTED_GRID": "512", "XCCL_MC_ROCM_DIRECT_TAIL": "0"})
    assert c["small_4src_stream"]["route"] == "tail" and c["small_4src_own"]["route"] == "stream"
    assert c["four_tiles_own"]["route"] == "slots"
    t = _routes({"XCCL_MC_ROCM_TAIL_FLAG": "0"})
    assert t["mid_stream"]["route"] == "counted" and t["large_stream"]["route"] == "stream"
    assert t["mid_own"] == d["mid_own"]
    r = _routes({"XCCL_MC_ROCM_RESIDENT_PER_CU": "8"})
    assert r["huge_stream"]["lds_bytes"] == 20480 and r["large_stream"]["lds_bytes"] == 20480
    assert r["small_4src_stream"]["lds_bytes"] == 0    # the whole grid is resident anyway
    r = _routes({"XCCL_MC_ROCM_RESIDENT_PER_CU": "32"})
    assert r["huge_stream"]["lds_bytes"] == 0
    b = _routes({"XCCL_MC_ROCM_BLOCKS_PER_CU": "4"})
    cap = b["huge_stream"]["grid"]                      # 4 x the device's compute units
    assert cap % 4 == 0 and 4 <= cap < 4096 and b["large_stream"]["grid"] == cap and b["mid_stream"]["grid"] == cap
    assert b["small_4src_stream"]["grid"] == 1000 and b["mid_own"]["route"] == "tail"
    assert _routes({"XCCL_MC_ROCM_BLOCKS_PER_CU": "8"})["huge_stream"]["grid"] == 2 * cap
    u = _routes({"XCCL_MC_ROCM_BURST_MAX_GRID": "0"})
    assert not u["four_tiles_stream"]["burst"] and not u["small_4src_own"]["burst"]
    u = _routes({"XCCL_MC_ROCM_BURST_MAX_GRID": "5000"})
    assert u["mid_own"]["burst"] and not u["large_own"]["burst"]
    s = _routes({"XCCL_MC_ROCM_SLOT_MAX_GRID": "0"})
    assert s["four_tiles_stream"]["route"] == "counted" and s["four_tiles_own"]["route"] == "counted"
    g = _routes({"XCCL_MC_ROCM_DIRECT_SIGNAL": "1", "XCCL_MC_ROCM_DIRECT_TAIL": "0"})
    assert g["large_own"]["route"] == "signal" and g["huge_own"]["route"] == "signal" and g["mid_own"]["route"] == "counted"
    assert g["large_stream"] == d["large_stream"]
    assert _routes({"XCCL_MC_ROCM_DIRECT_SIGNAL": "1"})["large_own"]["route"] == "tail"         # the second packet comes first
