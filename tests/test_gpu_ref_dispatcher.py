"""The plugin driven by the REFERENCE'S OWN dispatcher, not by this
repository's restatement of it: reference src/utils/mem_component.c, compiled
as it lies (and once more with integration/xccl-rocm.patch applied) by
tests/refdispatch/Makefile, dlopens xccl_rocm_mem_component.so the way libxccl
would and calls through the vtable (mem_component.c:11-49,51-148,231-283).
Results are compared with the CPU oracle.

Each variant runs in a process of its own: the reference loader writes the
vtable's `dlhandle` and `cache` members and its free_cache() closes the
component, which must not happen under the feet of the other tests' dispatcher.
Skipped where the two objects are not built (they are compiled in the
container that holds the reference tree and travel as built files)."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILD = os.path.join(ROOT, "tests", "refdispatch", "_build")
VARIANTS = {"unpatched": os.path.join(BUILD, "libref_mc_unpatched.so"),
            "patched": os.path.join(BUILD, "libref_mc_patched.so")}


def _drive(variant):
    """Runs in the child process; raises on the first difference."""
    import ctypes

    import numpy as np

    sys.path.insert(0, ROOT)
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from gpu_util import NP, assert_same
    from oracle import pyoracle as o
    from xccl_amd import hip, mc
    from xccl_amd.build import LIB_DIR
    from xccl_amd.types import Dt, MemType, Op, Status, StreamType, dt_size

    patched = variant == "patched"
    hip.set_device(0)
    os.environ["XCCL_MEM_COMPONENT_CACHE_SIZE"] = "4096"
    ref = mc.bind_dispatcher(VARIANTS[variant])
    assert hasattr(ref, "xccl_mem_component_reduce_multi_nb") == patched
    assert not hasattr(ref, "xccl_mem_component_get"), "this is not the reference's dispatcher"

    # mem_component.c:11-49 -- file name from ucs_memory_type_names[], symbol "xccl_cuda_mem_component"
    # (unpatched: the alias) or the component's own name (patched)
    assert ref.xccl_mem_component_init(LIB_DIR.encode()) == Status.OK
    comp = mc.component()                         # the same object, seen from outside
    assert comp.super.dlhandle, "the loader did not take the component"
    assert comp.super.cache.size == 4096 and comp.super.cache.used == 0 and not comp.super.cache.buf

    def mem_type(ptr):
        mt = ctypes.c_int(-1)
        st = ref.xccl_mem_component_type(ptr, ctypes.byref(mt))
        return st, mt.value

    def alloc(n):
        p = ctypes.c_void_p()
        st = ref.xccl_mem_component_alloc(ctypes.byref(p), n, int(MemType.ROCM))
        return st, p.value

    # mem_component.c:150-174
    dev = hip.DeviceBuffer(1 << 16)
    assert mem_type(dev.ptr) == (Status.OK, MemType.ROCM) and mem_type(dev.ptr + 4097) == (Status.OK, MemType.ROCM)
    plain = ctypes.create_string_buffer(64)
    assert mem_type(ctypes.addressof(plain)) == (Status.OK, MemType.HOST)
    pinned = hip.host_malloc(4096)
    assert mem_type(pinned) == (Status.OK, MemType.HOST)
    hip.host_free(pinned)
    dev.close()

    # mem_component.c:51-105 -- the one cached buffer
    st, p1 = alloc(1000)
    assert st == Status.OK and p1 == comp.super.cache.buf and comp.super.cache.used == 1
    st, p2 = alloc(1000)
    assert st == Status.OK and p2 != p1
    assert ref.xccl_mem_component_free(p1, int(MemType.ROCM)) == Status.OK and comp.super.cache.used == 0
    st, p3 = alloc(4096)
    assert st == Status.OK and p3 == p1
    st, p4 = alloc(4097)
    assert st == Status.OK and p4 not in (p1, p2)
    for p in (p2, p3, p4):
        assert ref.xccl_mem_component_free(p, int(MemType.ROCM)) == Status.OK
    assert comp.super.cache.used == 0 and comp.super.cache.buf == p1

    # mem_component.c:107-148 -- reduce, reduce_multi, size == 0
    def case(dt, op, nsrc, size, seed):
        es = dt_size(dt)
        slab = o.slab(nsrc, size, dt, seed, sparse=op in (Op.LAND, Op.LOR, Op.LXOR))
        st, buf = alloc((nsrc + 1) * size * es)          # scratch the way the call sites get it
        assert st == Status.OK
        hip.memcpy_htod(buf, slab)
        want = np.empty(size, dtype=slab.dtype)
        o.reduce_multi(slab, slab, want, nsrc - 1, size, size * es, dt, op, off2=size * es)
        return slab, buf, buf + size * es, buf + nsrc * size * es, want

    def result(ptr, size, dt):
        out = np.empty(size, dtype=NP[int(dt)])
        hip.memcpy_dtoh(out, ptr)
        return out

    n_calls = 0
    for dt, op, nsrc, size in ((Dt.INT32, Op.SUM, 4, 32), (Dt.FLOAT32, Op.SUM, 8, 1 << 18), (Dt.INT8, Op.MAX, 3, 100003),
                               (Dt.UINT16, Op.LXOR, 5, 4099), (Dt.INT64, Op.BXOR, 2, 777), (Dt.FLOAT16, Op.PROD, 4, 513),
                               (Dt.FLOAT64, Op.MIN, 16, 1 << 16), (Dt.UINT64, Op.PROD, 4, 1 << 20)):
        slab, p1, p2, pr, want = case(dt, op, nsrc, size, seed=7 + n_calls)
        es = dt_size(dt)
        st = ref.xccl_mem_component_reduce_multi(p1, p2, pr, nsrc - 1, size, size * es, int(dt), int(op), int(MemType.ROCM))
        assert st == Status.OK, (dt, op, st)
        assert_same(result(pr, size, dt), want, dt, op, "%s reduce_multi %s %s" % (variant, dt.name, op.name))
        # the 2-source entry, in place on sbuf2 (reduce_linear.c:28-34)
        two = np.empty(size, dtype=slab.dtype)
        o.dt_reduce(slab[0], slab[1], two, size, dt, op)
        st = ref.xccl_mem_component_reduce(p1, p2, p2, size, int(dt), int(op), int(MemType.ROCM))
        assert st == Status.OK
        assert_same(result(p2, size, dt), two, dt, op, "%s reduce %s %s" % (variant, dt.name, op.name))
        # size == 0: XCCL_OK, nothing touched (mem_component.c:129-131)
        st = ref.xccl_mem_component_reduce_multi(p1, p2, pr, nsrc - 1, 0, size * es, int(dt), int(op), int(MemType.ROCM))
        assert st == Status.OK
        assert_same(result(pr, size, dt), want, dt, op, "size == 0 wrote something")
        assert ref.xccl_mem_component_free(p1, int(MemType.ROCM)) == Status.OK
        n_calls += 1
    # what neither the reference nor the component implements
    st, buf = alloc(4096)
    assert ref.xccl_mem_component_reduce(buf, buf, buf, 4, int(Dt.FLOAT32), int(Op.BAND), int(MemType.ROCM)) == \
        Status.ERR_UNSUPPORTED
    assert ref.xccl_mem_component_reduce_multi(buf, buf, buf, 1, 4, 16, int(Dt.INT128), int(Op.SUM),
                                               int(MemType.ROCM)) == Status.ERR_UNSUPPORTED
    assert ref.xccl_mem_component_free(buf, int(MemType.ROCM)) == Status.OK

    if patched:
        # the entries and the stream type only the patched dispatcher has
        # (mem_component.c:176-178,231-257 + the patch's reduce_nb / reduce_multi_nb)
        hs = hip.stream_create()
        s = mc.Stream(hs, StreamType.ROCM)
        ev = ctypes.c_void_p()
        assert ref.xccl_mc_event_record(s.ref(), ctypes.byref(ev)) == Status.OK and ev.value
        assert ctypes.c_int.from_address(ev.value).value == MemType.ROCM
        while True:
            st = ref.xccl_mc_event_query(ev)
            assert st in (Status.OK, Status.INPROGRESS)
            if st == Status.OK:
                break
        assert ref.xccl_mc_event_free(ev) == Status.OK
        for dt, op, nsrc, size in ((Dt.FLOAT32, Op.SUM, 4, 256), (Dt.INT32, Op.MIN, 8, 1 << 20),
                                   (Dt.FLOAT64, Op.SUM, 3, 1 << 22)):
            slab, p1, p2, pr, want = case(dt, op, nsrc, size, seed=31)
            es = dt_size(dt)
            ev = ctypes.c_void_p()
            st = ref.xccl_mem_component_reduce_multi_nb(p1, p2, pr, nsrc - 1, size, size * es, int(dt), int(op),
                                                        int(MemType.ROCM), None, ctypes.byref(ev))
            assert st == Status.OK and ev.value and ctypes.c_int.from_address(ev.value).value == MemType.ROCM
            while ref.xccl_mc_event_query(ev) == Status.INPROGRESS:
                pass
            assert ref.xccl_mc_event_query(ev) == Status.OK and ref.xccl_mc_event_free(ev) == Status.OK
            assert_same(result(pr, size, dt), want, dt, op, "patched reduce_multi_nb %s %s" % (dt.name, op.name))
            # on the caller's stream, no event: ordered before the copy queued behind it
            two = np.empty(size, dtype=slab.dtype)
            o.dt_reduce(slab[2], slab[1], two, size, dt, op)
            st = ref.xccl_mem_component_reduce_nb(p1 + 2 * size * es, p2, pr, size, int(dt), int(op),
                                                  int(MemType.ROCM), s.ref(), None)
            assert st == Status.OK
            assert ref.xccl_mem_component_memcpy_async(pr, p1, size * es, s.ref()) == Status.OK
            hip.stream_synchronize(hs)
            assert_same(result(p1, size, dt), two, dt, op, "patched reduce_nb on a stream %s %s" % (dt.name, op.name))
            # an empty reduction is complete on return
            ev = ctypes.c_void_p(1)
            st = ref.xccl_mem_component_reduce_multi_nb(p1, p2, pr, nsrc - 1, 0, size * es, int(dt), int(op),
                                                        int(MemType.ROCM), None, ctypes.byref(ev))
            assert st == Status.OK and not ev.value
            assert ref.xccl_mem_component_free(p1, int(MemType.ROCM)) == Status.OK
        # the event pool runs dry: the dispatcher's fallback is the blocking entry (event NULL, result there)
        held = []
        while True:
            e = ctypes.c_void_p()
            st = ref.xccl_mc_event_record(s.ref(), ctypes.byref(e))
            if st != Status.OK:
                assert st == Status.ERR_NO_RESOURCE
                break
            held.append(e)
            assert len(held) <= 4096
        slab, p1, p2, pr, want = case(Dt.INT32, Op.SUM, 4, 1000, seed=5)
        ev = ctypes.c_void_p(1)
        st = ref.xccl_mem_component_reduce_multi_nb(p1, p2, pr, 3, 1000, 4000, int(Dt.INT32), int(Op.SUM),
                                                    int(MemType.ROCM), None, ctypes.byref(ev))
        assert st == Status.OK and not ev.value
        assert_same(result(pr, 1000, Dt.INT32), want, Dt.INT32, Op.SUM, "fallback to the blocking entry")
        st = ref.xccl_mem_component_reduce_multi_nb(p1, p2, pr, 3, 1000, 4000, int(Dt.INT32), int(Op.SUM),
                                                    int(MemType.ROCM), s.ref(), ctypes.byref(ev))
        assert st == Status.ERR_NO_RESOURCE
        for e in held:
            assert ref.xccl_mc_event_free(e) == Status.OK
        assert ref.xccl_mem_component_free(p1, int(MemType.ROCM)) == Status.OK
        # stream gate through the patched stream table (mem_component.c:197-229)
        req = ctypes.c_void_p()
        assert ref.xccl_mem_component_start_acitivity(s.ref(), ctypes.byref(req)) == Status.OK
        assert ctypes.c_int.from_address(req.value).value == MemType.ROCM
        assert ref.xccl_mem_component_finish_acitivity(req) == Status.OK
        hip.stream_synchronize(hs)
        hip.stream_destroy(hs)

    # mem_component.c:259-283
    assert comp.super.cache.buf and comp.super.cache.used == 0
    ref.xccl_mem_component_free_cache()
    ref.xccl_mem_component_finalize()
    print("ref-dispatcher %s ok: %d (dtype, op) cases" % (variant, n_calls), flush=True)


@pytest.mark.gpu
@pytest.mark.parametrize("variant", sorted(VARIANTS))
def test_reference_dispatcher_drives_the_plugin(variant):
    if not os.path.isfile(VARIANTS[variant]):
        pytest.skip("%s not built (make -C tests/refdispatch needs the reference tree)" % VARIANTS[variant])
    out = subprocess.run([sys.executable, "-u", os.path.abspath(__file__), variant], capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0 and "ref-dispatcher %s ok" % variant in out.stdout, out.stdout + out.stderr


if __name__ == "__main__":
    _drive(sys.argv[1])
