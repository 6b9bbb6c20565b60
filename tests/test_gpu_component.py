"""The rest of the component's vtable on a real device: memory-type probing,
the dispatcher's buffer cache on device memory, events and their pool,
stream-ordered reductions, the graph launch path, the stream gate, and the
synthetic-input kernels against the oracle's generator."""
import ctypes
import time

import numpy as np
import pytest

from gpu_util import NP, Case, assert_same
from xccl_amd import hip
from xccl_amd.types import Dt, MemType, Op, Status, StreamType, dt_size

pytestmark = pytest.mark.gpu


def test_mem_type_probe(rocm):
    """cuda_mem_component.c:182-204: device memory -> the component's type,
    pinned host memory -> HOST, ordinary host memory -> HOST (component says
    UNSUPPORTED, dispatcher falls through), and the runtime is left without a
    sticky error."""
    d = hip.DeviceBuffer(1024)
    assert rocm.xccl_mem_component_type(d.ptr) == (Status.OK, MemType.ROCM)
    assert rocm.xccl_mem_component_type(d.ptr + 512) == (Status.OK, MemType.ROCM)
    pinned = hip.host_malloc(1024)
    assert rocm.xccl_mem_component_type(pinned) == (Status.OK, MemType.HOST)
    # managed memory is not "Device" to the runtime: HOST, like in the reference (cuda_mem_component.c:198-202)
    managed = hip.malloc_managed(1 << 16)
    assert rocm.xccl_mem_component_type(managed) == (Status.OK, MemType.HOST)
    assert rocm.xccl_mem_component_type(managed + 12345) == (Status.OK, MemType.HOST)
    mt = ctypes.c_int(-1)
    assert rocm.component().super.mem_type(managed + 4096, ctypes.byref(mt)) == Status.OK and mt.value == MemType.HOST
    hip.free(managed)
    plain = ctypes.create_string_buffer(64)
    assert rocm.xccl_mem_component_type(ctypes.addressof(plain)) == (Status.OK, MemType.HOST)
    mt = ctypes.c_int(-1)
    st = rocm.component().super.mem_type(ctypes.addressof(plain), ctypes.byref(mt))
    assert st in (Status.ERR_UNSUPPORTED, Status.OK)
    assert hip.lib().hipGetLastError() == 0
    hip.host_free(pinned)
    d.close()


def test_device_alloc_cache(rocm):
    """mem_component.c:51-105 on the real component: a request that fits the
    4 KiB cache gets the cached device buffer, a second concurrent one and an
    oversized one get their own."""
    st, p1 = rocm.xccl_mem_component_alloc(3 * 1024, MemType.ROCM)
    assert st == Status.OK and rocm.xccl_mem_component_type(p1) == (Status.OK, MemType.ROCM)
    st, p2 = rocm.xccl_mem_component_alloc(3 * 1024, MemType.ROCM)
    assert st == Status.OK and p2 != p1
    assert rocm.xccl_mem_component_free(p1, MemType.ROCM) == Status.OK
    st, p3 = rocm.xccl_mem_component_alloc(4096, MemType.ROCM)
    assert p3 == p1
    st, p4 = rocm.xccl_mem_component_alloc(1 << 20, MemType.ROCM)
    assert st == Status.OK and p4 not in (p1, p2)
    for p in (p2, p3, p4):
        assert rocm.xccl_mem_component_free(p, MemType.ROCM) == Status.OK


def test_freed_scratch_is_cached_and_reused(rocm, oracle):
    """The component's mem_free keeps blocks for the next mem_alloc of the same
    size class (per-collective scratch, allreduce_knomial.c:181-183), a reused
    block works as reduction scratch, and a limit of 0 restores the runtime's
    allocate/free per call."""
    MiB = 1 << 20
    comp = rocm.component()
    rocm.mem_pool_set_limit(0)                      # start from an empty cache
    rocm.mem_pool_set_limit(64 * MiB)
    s0 = rocm.mem_pool_stats()

    def alloc(n):
        p = ctypes.c_void_p()
        assert comp.super.mem_alloc(ctypes.byref(p), n) == Status.OK
        return p.value

    a = alloc(3 * MiB)
    assert rocm.xccl_mem_component_type(a) == (Status.OK, MemType.ROCM)
    assert comp.super.mem_free(a) == Status.OK
    s1 = rocm.mem_pool_stats()
    assert s1.free_blocks == 1 and s1.cached_bytes == 3 * MiB and s1.misses == s0.misses + 1
    b = alloc(3 * MiB - 100)                        # same class: the same block
    assert b == a and rocm.mem_pool_stats().hits == s0.hits + 1
    c = alloc(3 * MiB)                              # a second one while the first is live
    assert c != a

    # the reused block as scratch of a 4-source reduce_multi (3 vectors at stride 1 MiB)
    n = 200_000
    s1 = oracle.fill(n, Dt.INT32, 21, 1000)
    s2 = np.zeros((3, MiB // 4), dtype=np.int32)
    for j in range(3):
        s2[j, :n] = oracle.fill(n, Dt.INT32, 21, j)
    want = np.empty(n, dtype=np.int32)
    oracle.reduce_multi(s1, s2, want, 3, n, MiB, Dt.INT32, Op.SUM)
    own = hip.DeviceBuffer(n * 4)
    dst = hip.DeviceBuffer(n * 4)
    own.upload(s1)
    hip.memcpy_htod(b, s2)
    assert rocm.xccl_mem_component_reduce_multi(own.ptr, b, dst.ptr, 3, n, MiB, Dt.INT32, Op.SUM,
                                                MemType.ROCM) == Status.OK
    assert_same(dst.download(np.int32, n, 0), want, Dt.INT32, Op.SUM, "reduction out of a reused scratch block")

    assert comp.super.mem_free(b) == Status.OK and comp.super.mem_free(c) == Status.OK
    assert comp.super.mem_free(b) == Status.ERR_NO_MESSAGE          # freed twice: reported, nothing released
    assert rocm.mem_pool_stats().free_blocks == 2
    big = alloc(128 * MiB)                          # beyond the limit: never kept
    assert comp.super.mem_free(big) == Status.OK
    assert rocm.mem_pool_stats().free_blocks == 2
    rocm.mem_pool_set_limit(0)
    s2 = rocm.mem_pool_stats()
    assert s2.free_blocks == 0 and s2.cached_bytes == 0 and s2.live_blocks == s0.live_blocks
    d = alloc(3 * MiB)
    assert comp.super.mem_free(d) == Status.OK
    assert rocm.mem_pool_stats().hits == s0.hits + 1                # nothing was served from a cache
    rocm.mem_pool_set_limit(8 << 30)
    own.close()
    dst.close()


def test_event_record_query_free_and_pool(rocm):
    """Pool exhaustion is XCCL_ERR_NO_RESOURCE (cuda_mem_component.c:91,107);
    a freed slot is reusable."""
    s = rocm.Stream(hip.stream_create())
    evs = []
    while True:
        st, ev = rocm.xccl_mc_event_record(s)
        if st != Status.OK:
            break
        evs.append(ev)
        assert len(evs) <= 4096
    assert st == Status.ERR_NO_RESOURCE and len(evs) == 64
    hip.stream_synchronize(s.hip_stream)
    for ev in evs:
        assert ctypes.c_int.from_address(ev).value == MemType.ROCM
        assert rocm.xccl_mc_event_query(ev) == Status.OK
        assert rocm.xccl_mc_event_free(ev) == Status.OK
    st, ev = rocm.xccl_mc_event_record(s)
    assert st == Status.OK
    assert rocm.xccl_mc_event_wait(ev) == Status.OK
    assert rocm.xccl_mc_event_free(ev) == Status.OK
    hip.stream_destroy(s.hip_stream)


@pytest.mark.parametrize("own_stream", [False, True])
def test_stream_ordered_reduce_multi(rocm, oracle, own_stream):
    """reduce_multi_nb returns with the kernel enqueued; the event turns from
    INPROGRESS/OK to OK and the result is then complete.  Two dependent calls
    on one stream (round k's rbuf is round k+1's sbuf1, allreduce_knomial.c:
    118-135) need no host wait in between."""
    dt, op, size, n2 = Dt.FLOAT32, Op.SUM, 1 << 22, 3
    c = Case(dt, size, n2)
    s = rocm.Stream(hip.stream_create()) if own_stream else None
    try:
        c.fill_random(oracle, 12)
        c.upload()
        p1, p2, pr = c.ptrs()
        st, ev1 = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, n2, size, c.stride, dt, op, MemType.ROCM, s)
        assert st == Status.OK and ev1
        st, ev2 = rocm.xccl_mem_component_reduce_multi_nb(pr, p2, pr, n2, size, c.stride, dt, op, MemType.ROCM, s)
        assert st == Status.OK and ev2
        t0 = time.time()
        while True:
            q = rocm.xccl_mc_event_query(ev2)
            if q == Status.OK:
                break
            assert q == Status.INPROGRESS and time.time() - t0 < 30
        assert rocm.xccl_mc_event_query(ev1) == Status.OK
        img = c.host.copy()
        b = img.ctypes.data
        oracle.reduce_multi_ptr(b + c.o1, b + c.o2, b + c.orr, n2, size, c.stride, dt, op)
        oracle.reduce_multi_ptr(b + c.orr, b + c.o2, b + c.orr, n2, size, c.stride, dt, op)
        assert_same(c.result(), img[c.orr: c.orr + c.vbytes], dt, op, "nb chain")
        assert rocm.xccl_mc_event_free(ev1) == Status.OK and rocm.xccl_mc_event_free(ev2) == Status.OK
        # without an event: completion through the stream itself
        st, ev = rocm.xccl_mem_component_reduce_nb(p1, p2, pr, size, dt, op, MemType.ROCM, s, want_event=False)
        assert st == Status.OK and not ev
        hip.stream_synchronize(s.hip_stream if s else rocm.component_stream())
        want = np.empty(size, dtype=np.float32)
        oracle.dt_reduce(c.host[c.o1:c.o1 + c.vbytes].view(np.float32), c.host[c.o2:c.o2 + c.vbytes].view(np.float32),
                         want, size, dt, op)
        assert_same(c.result(), want.view(np.uint8), dt, op, "reduce_nb")
        # unsupported pair: status, no event consumed
        st, ev = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, n2, size, c.stride, dt, Op.BAND, MemType.ROCM, s)
        assert st == Status.ERR_UNSUPPORTED and not ev
    finally:
        c.close()
        if s:
            hip.stream_destroy(s.hip_stream)


def test_graph_launch_matches_plain_launch(rocm, oracle):
    """The single-node graph path: same bits as the plain launch, across cache
    hits (same arguments replayed), parameter patches (more argument sets than
    cache slots) and several replays with other work in between."""
    lib = rocm.component_lib()
    stream = rocm.component_stream()
    dt, op = Dt.FLOAT32, Op.SUM
    cases = []
    try:
        for k in range(11):                      # > 8 cache slots
            c = Case(dt, 64 + 257 * k, 1 + k % 4, off2=4 * (k % 3))
            c.fill_random(oracle, 30 + k)
            c.upload()
            cases.append(c)
        for rep in range(3):
            for c in cases:
                p1, p2, pr = c.ptrs()
                hip.memset(pr, 0xEE, c.vbytes)
                st = lib.xccl_rocm_reduce_multi_graph(p1, p2, pr, c.n2, c.size, c.stride, int(dt), int(op), stream)
                assert st == Status.OK
                if rep == 1:                     # immediate replay: cache hit
                    assert lib.xccl_rocm_reduce_multi_graph(p1, p2, pr, c.n2, c.size, c.stride, int(dt), int(op),
                                                            stream) == Status.OK
                hip.stream_synchronize(stream)
                want, _ = c.expect(oracle, op)
                assert_same(c.result(), want, dt, op, "graph rep %d size %d" % (rep, c.size))
            # eager work between rounds of replays
            run = cases[0]
            p1, p2, pr = run.ptrs()
            assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, run.n2, run.size, run.stride, dt, op,
                                                        MemType.ROCM) == Status.OK
        assert lib.xccl_rocm_reduce_multi_graph(p1, p2, pr, 1, 16, 64, int(dt), int(Op.BAND), stream) \
            == Status.ERR_UNSUPPORTED
    finally:
        for c in cases:
            c.close()
        lib.xccl_rocm_graph_cache_destroy()


def test_memcpy_async_source_first(rocm):
    """mem_component.h:38: (sbuf, dbuf, size, stream) -- source first."""
    s = rocm.Stream(hip.stream_create())
    a = hip.DeviceBuffer(4096)
    b = hip.DeviceBuffer(4096)
    data = np.arange(1024, dtype=np.uint32)
    a.upload(data)
    hip.memset(b.ptr, 0, 4096)
    assert rocm.xccl_mem_component_memcpy_async(a.ptr, b.ptr, 4096, s) == Status.OK
    hip.stream_synchronize(s.hip_stream)
    assert np.array_equal(b.download(np.uint32, 1024), data)
    hip.stream_destroy(s.hip_stream)
    a.close()
    b.close()


def test_stream_activity_gate(rocm):
    """cuda_mem_component.c:139-180: work enqueued on the user stream after
    start_stream_activity does not run until finish_stream_activity.  The gate
    kernel's wait is bounded, so nothing here can hang the queue."""
    s = rocm.Stream(hip.stream_create())
    a = hip.DeviceBuffer(4096)
    b = hip.DeviceBuffer(4096)
    a.upload(np.full(1024, 7, dtype=np.uint32))
    hip.memset(b.ptr, 0, 4096)
    st, req = rocm.xccl_mem_component_start_acitivity(s)
    assert st == Status.OK and ctypes.c_int.from_address(req).value == MemType.ROCM
    assert rocm.xccl_mem_component_memcpy_async(a.ptr, b.ptr, 4096, s) == Status.OK
    st, ev = rocm.xccl_mc_event_record(s)
    assert st == Status.OK
    time.sleep(0.2)
    assert rocm.xccl_mc_event_query(ev) == Status.INPROGRESS      # still gated
    # a blocking reduction issued while the gate is shut (a host-progressed collective doing its
    # arithmetic) must not queue up behind the gate
    t0 = time.time()
    assert rocm.xccl_mem_component_reduce(a.ptr, a.ptr + 2048, a.ptr + 2048, 512, Dt.UINT32, Op.SUM,
                                          MemType.ROCM) == Status.OK
    assert time.time() - t0 < 5.0
    assert rocm.xccl_mc_event_query(ev) == Status.INPROGRESS
    assert rocm.xccl_mem_component_finish_acitivity(req) == Status.OK
    assert rocm.xccl_mc_event_wait(ev) == Status.OK
    # read back only now: a copy issued while the gate is shut may be given the hardware queue the gated stream
    # sits on (HIP shares a few among all streams) and would then wait for the gate
    assert (a.download(np.uint32, 512, 2048) == 14).all()
    assert (b.download(np.uint32, 1024)[:512] == 7).all()
    assert rocm.xccl_mc_event_free(ev) == Status.OK
    # slots recycle: more start/finish pairs than the pool holds
    for _ in range(10):
        st, req = rocm.xccl_mem_component_start_acitivity(s)
        assert st == Status.OK
        assert rocm.xccl_mem_component_finish_acitivity(req) == Status.OK
        hip.stream_synchronize(s.hip_stream)
    hip.stream_destroy(s.hip_stream)
    a.close()
    b.close()


def test_stream_gate_times_out_by_itself(rocm):
    """A gate nobody opens leaves after its time limit and marks the word with
    2 (forced from the host with a 50 ms limit; no wave is left spinning)."""
    lib = rocm.component_lib()
    flag_host = hip.host_malloc(64)
    ctypes.c_int.from_address(flag_host).value = 0
    dev = ctypes.c_void_p()
    hip.check(hip.lib().hipHostGetDevicePointer(ctypes.byref(dev), ctypes.c_void_p(flag_host), 0))
    stream = rocm.component_stream()
    t0 = time.time()
    assert lib.xccl_rocm_stream_gate(dev, 50 * 1000 * 1000, stream) == Status.OK
    hip.stream_synchronize(stream)
    dt = time.time() - t0
    assert ctypes.c_int.from_address(flag_host).value == 2
    assert 0.03 < dt < 5.0
    hip.host_free(flag_host)


def test_finish_stream_activity_reports_a_gate_that_gave_up():
    """A gate whose time limit passes before finish_stream_activity let the
    user's stream run early; finish must say so (XCCL_ERR_NO_PROGRESS) instead
    of returning XCCL_OK.  The limit comes from the environment, read once per
    process, hence a child process with a 30 ms limit; the gate kernel leaves
    by itself, nothing is left spinning."""
    import os
    import subprocess
    import sys
    code = (
        "import sys, time\n"
        "sys.path.insert(0, %r)\n"
        "from xccl_amd import hip, mc\n"
        "from xccl_amd.types import Status\n"
        "hip.set_device(0)\n"
        "assert mc.xccl_mem_component_init() == Status.OK\n"
        "s = mc.Stream(hip.stream_create())\n"
        "st, req = mc.xccl_mem_component_start_acitivity(s)\n"
        "assert st == Status.OK\n"
        "hip.stream_synchronize(s.hip_stream)\n"       # returns once the gate has given up
        "late = mc.xccl_mem_component_finish_acitivity(req)\n"
        "st, req = mc.xccl_mem_component_start_acitivity(s)\n"
        "assert st == Status.OK\n"
        "in_time = mc.xccl_mem_component_finish_acitivity(req)\n"
        "hip.stream_synchronize(s.hip_stream)\n"
        "print('late', int(late), 'in_time', int(in_time))\n"
    ) % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, XCCL_MC_ROCM_GATE_TIMEOUT_MS="30")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "late %d in_time %d" % (int(Status.ERR_NO_PROGRESS), int(Status.OK)) in out.stdout, out.stdout + out.stderr
    assert "stream gate gave up" in out.stderr


@pytest.mark.parametrize("dt", [Dt.INT8, Dt.UINT16, Dt.INT32, Dt.UINT64, Dt.FLOAT16, Dt.FLOAT32, Dt.FLOAT64],
                         ids=lambda d: Dt(d).name)
def test_datagen_matches_oracle_generator(rocm, oracle, dt):
    """The GPU input generator and the oracle's CPU generator follow one
    recipe: identical bits for integers, binary16 and binary32; binary64 goes
    through log/cos of two different math libraries and agrees to 1e-13."""
    n = 100003
    d = hip.DeviceBuffer(n * dt_size(dt))
    for sparse in (False, True):
        assert rocm.datagen_fill(d.ptr, n, dt, 5, 3, sparse) == Status.OK
        hip.device_synchronize()
        got = d.download(NP[int(dt)], n)
        want = oracle.fill(n, dt, 5, 3, sparse)
        if dt == Dt.FLOAT64:
            assert np.allclose(got, want, rtol=0, atol=1e-13)
        else:
            assert got.tobytes() == want.tobytes()
    d.close()


def test_completion_word_threshold_and_sequences(rocm, oracle):
    """Completion through a host-mapped word: written by the launch itself
    (up to 1024 workgroups of 512 floats here, up to 8192 when the result has
    peeled head/tail elements), by a one-lane kernel queued behind a larger
    launch without such elements, and not at all beyond (then the stream is
    waited for).  Sizes on every side of those switches, grids that fill the
    64 arrival-counter shards unevenly (65, 100, 129, 1000 workgroups), many
    back-to-back blocking calls (sequence numbers advance per pooled event),
    results checked every time."""
    dt, op = Dt.FLOAT32, Op.SUM
    tile = 512
    for size in (1, 63, 64 * tile, 65 * tile, 100 * tile + 3, 129 * tile - 1, 1000 * tile + 17, 1024 * tile,
                 1025 * tile, 2048 * tile + 4, 8192 * tile - 1, 8192 * tile, 8192 * tile + 1, 8193 * tile + 5,
                 20000 * tile):
        c = Case(dt, size, 1)
        try:
            c.fill_random(oracle, 21)
            c.upload()
            p1, p2, pr = c.ptrs()
            want, _ = c.expect(oracle, op)
            for rep in range(5):
                hip.memset(pr, 0x11 * (rep + 1), c.vbytes)
                assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, 1, size, c.stride, dt, op,
                                                            MemType.ROCM) == Status.OK
                assert_same(c.result(), want, dt, op, "size %d rep %d" % (size, rep))
        finally:
            c.close()
    # 300 blocking calls in a row on a tiny message: every one must be complete on return
    c = Case(Dt.INT32, 64, 3)
    try:
        c.fill_random(oracle, 22)
        c.upload()
        p1, p2, pr = c.ptrs()
        want, _ = c.expect(oracle, Op.SUM)
        for rep in range(300):
            assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, 3, 64, c.stride, Dt.INT32, Op.SUM,
                                                        MemType.ROCM) == Status.OK
            if rep % 50 == 0:
                assert_same(c.result(), want, Dt.INT32, Op.SUM, "rep %d" % rep)
    finally:
        c.close()


def test_completion_by_one_word_per_workgroup(rocm, oracle):
    """Launches of a handful of workgroups (2 to 8 by default, up to 16 on
    request) report completion without counting: workgroup b stores the
    sequence number to word b of the caller's 16 words.  Through the C ABI:
    the number of words to watch comes back in `flagged`, each of them ends up
    holding the sequence number, words beyond keep what they held, and the
    result is the oracle's; a caller with too few words, a launch of one
    workgroup and one beyond the bound get the counting path (`flagged` 1).
    Then the same shapes through the component's blocking entry and
    reduce_multi_nb + event_query, with the path switched off and on."""
    lib = rocm.component_lib()
    stream = rocm.component_stream()
    words = 16
    host = hip.host_malloc(4 * words)
    ctypes.memset(host, 0, 4 * words)
    dev = hip.host_get_device_pointer(host)
    view = ctypes.cast(host, ctypes.POINTER(ctypes.c_uint32))
    counters = hip.malloc((1 + 64) * 128)
    hip.memset(counters, 0, (1 + 64) * 128)
    hip.device_synchronize()
    dt, op, n2 = Dt.FLOAT32, Op.SUM, 3
    seq = 0
    try:
        for bound, tiles, room, expect_words in ((-1, 1, 16, 1), (-1, 2, 16, 2), (-1, 7, 16, 7), (-1, 8, 16, 8),
                                                 (-1, 9, 16, 1), (16, 9, 16, 9), (16, 16, 16, 16), (16, 17, 16, 1),
                                                 (64, 17, 64, 1), (-1, 7, 1, 1), (-1, 7, 4, 1), (-1, 4, 4, 4),
                                                 (0, 4, 16, 1)):
            lib.xccl_rocm_set_slot_max_grid(bound)
            size = tiles * 256 - 3              # ragged last tile, peeled tail elements
            c = Case(dt, size, n2)
            try:
                c.fill_random(oracle, 90 + tiles)
                c.upload()
                p1, p2, pr = c.ptrs()
                want, _ = c.expect(oracle, op)
                hip.memset(pr, 0xAB, c.vbytes)
                hip.device_synchronize()
                before = [view[i] for i in range(words)]
                seq += 1
                flagged = ctypes.c_int(-1)
                st = lib.xccl_rocm_reduce_multi_slots(p1, p2, pr, n2, size, c.stride, int(dt), int(op), stream, counters,
                                                      dev, room, seq, ctypes.byref(flagged))
                assert st == Status.OK
                assert flagged.value == expect_words, (tiles, room, flagged.value)
                t0 = time.time()
                while any(view[i] != seq for i in range(flagged.value)):
                    assert time.time() - t0 < 20.0, "completion words never written: %s" % [view[i] for i in range(8)]
                assert_same(c.result(), want, dt, op, "%d tiles, room for %d words" % (tiles, room))
                hip.stream_synchronize(stream)
                assert [view[i] for i in range(flagged.value, words)] == before[flagged.value:], (tiles, room)
            finally:
                c.close()
        for max_grid in (0, -1, 16):
            lib.xccl_rocm_set_slot_max_grid(max_grid)
            for tiles in (2, 3, 7, 8, 9, 16, 17):
                size = tiles * 256 - 1
                c = Case(dt, size, n2)
                try:
                    c.fill_random(oracle, 190 + tiles)
                    c.upload()
                    p1, p2, pr = c.ptrs()
                    want, _ = c.expect(oracle, op)
                    for rep in range(3):
                        hip.memset(pr, 0x10 + rep, c.vbytes)
                        assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, n2, size, c.stride, dt, op,
                                                                    MemType.ROCM) == Status.OK
                        assert_same(c.result(), want, dt, op, "blocking, %d tiles, rep %d" % (tiles, rep))
                        hip.memset(pr, 0x20 + rep, c.vbytes)
                        st, ev = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, n2, size, c.stride, dt, op,
                                                                         MemType.ROCM, None)
                        assert st == Status.OK and ev is not None
                        t0 = time.time()
                        while rocm.xccl_mc_event_query(ev) == Status.INPROGRESS:
                            assert time.time() - t0 < 20.0
                        assert rocm.xccl_mc_event_query(ev) == Status.OK
                        assert_same(c.result(), want, dt, op, "event, %d tiles, rep %d" % (tiles, rep))
                        assert rocm.xccl_mc_event_free(ev) == Status.OK
                finally:
                    c.close()
    finally:
        lib.xccl_rocm_set_slot_max_grid(-1)
        hip.stream_synchronize(stream)
        hip.free(counters)
        hip.host_free(host)


def test_blocking_calls_take_the_components_own_queue(rocm, oracle):
    """A blocking reduction goes out on the component's own dispatch queue, not
    on a HIP stream -- a small one carrying its completion word, a large one
    with a one-lane kernel as a second packet behind it -- unless the path is
    switched off, the large form is switched off and the call is too large, or
    the calling thread has launches outstanding on its stream that the call
    has to stay behind.  The counter of such launches says which way a call
    went; the result is the oracle's every time."""
    lib = rocm.component_lib()
    dt, op, n2 = Dt.FLOAT32, Op.SUM, 3
    small, large = Case(dt, 5000, n2), Case(dt, 3 * 1024 * 1024, n2)

    def blocking(c, tag):
        p1, p2, pr = c.ptrs()
        hip.memset(pr, 0x5C, c.vbytes)
        hip.device_synchronize()
        before = lib.xccl_rocm_direct_launch_count()
        assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, n2, c.size, c.stride, dt, op, MemType.ROCM) == Status.OK
        assert_same(c.result(), c.expect(oracle, op)[0], dt, op, tag)
        return lib.xccl_rocm_direct_launch_count() - before

    try:
        for c in (small, large):
            c.fill_random(oracle, 33)
            c.upload()
        blocking(small, "whichever way: earlier tests may have left stream-ordered launches nobody waited for")
        assert blocking(small, "own queue") == 1
        assert blocking(small, "own queue again") == 1
        assert blocking(large, "12 MiB vectors: own queue, completion word from a second packet") == 1
        lib.xccl_rocm_set_direct_tail(0)
        assert blocking(large, "12 MiB vectors, second packet switched off: the stream") == 0
        lib.xccl_rocm_set_direct_tail(1)
        lib.xccl_rocm_set_direct_queue(0)
        assert blocking(small, "switched off") == 0
        assert blocking(large, "switched off") == 0
        lib.xccl_rocm_set_direct_queue(1)
        # a launch on the thread's stream that nobody has waited for (no event: nothing but the stream can tell when
        # it is over): the next blocking call stays behind it on the stream
        p1, p2, pr = large.ptrs()
        hip.memset(pr, 0x11, large.vbytes)
        hip.device_synchronize()
        st, ev = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, n2, large.size, large.stride, dt, op, MemType.ROCM,
                                                         None, want_event=False)
        assert st == Status.OK and ev is None
        assert blocking(small, "behind a launch on the stream") == 0
        assert_same(large.result(), large.expect(oracle, op)[0], dt, op, "the launch on the stream")   # stream order
        assert blocking(small, "own queue once the stream has been waited for") == 1
        # a large stream-ordered launch with an event takes the own queue; a blocking call behind it is ordered behind it
        hip.memset(pr, 0x12, large.vbytes)
        hip.device_synchronize()
        before = lib.xccl_rocm_direct_launch_count()
        st, ev = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, n2, large.size, large.stride, dt, op, MemType.ROCM,
                                                         None)
        assert st == Status.OK and ev is not None
        assert blocking(small, "behind a stream-ordered launch on the own queue") == 1
        assert lib.xccl_rocm_direct_launch_count() - before == 2
        assert rocm.xccl_mc_event_query(ev) == Status.OK        # queue order: it has completed as well
        assert rocm.xccl_mc_event_free(ev) == Status.OK
        assert_same(large.result(), large.expect(oracle, op)[0], dt, op, "the stream-ordered launch")
        # a small stream-ordered call, then a large one WITHOUT an event, which has to go to the stream: it is issued
        # only after the first has been waited for on the host, so the order of one thread's calls holds across both
        p1, p2, pr = small.ptrs()
        hip.memset(pr, 0x3D, small.vbytes)
        hip.device_synchronize()
        before = lib.xccl_rocm_direct_launch_count()
        st, ev_small = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, n2, small.size, small.stride, dt, op,
                                                               MemType.ROCM, None)
        assert st == Status.OK and ev_small is not None
        assert lib.xccl_rocm_direct_launch_count() - before == 1
        q1, q2, qr = large.ptrs()
        st, none = rocm.xccl_mem_component_reduce_multi_nb(q1, q2, qr, n2, large.size, large.stride, dt, op,
                                                           MemType.ROCM, None, want_event=False)
        assert st == Status.OK and none is None
        assert lib.xccl_rocm_direct_launch_count() - before == 1    # the large one went to the stream
        assert rocm.xccl_mc_event_query(ev_small) == Status.OK      # and was issued only after the small one
        assert_same(small.result(), small.expect(oracle, op)[0], dt, op, "stream-ordered call on the own queue")
        assert rocm.xccl_mc_event_free(ev_small) == Status.OK
        assert blocking(small, "behind the launch on the stream") == 0
        assert_same(large.result(), large.expect(oracle, op)[0], dt, op, "the large launch on the stream")
        assert blocking(small, "own queue: the large launch has been seen complete") == 1
        # 48 stream-ordered calls in place, none waited for until the end: the queue runs them in order
        chain = Case(Dt.INT32, 3000, 1, alias="s1")
        try:
            chain.fill_random(oracle, 44, Op.SUM)
            chain.upload()
            c1, c2, cr = chain.ptrs()
            assert cr == c1
            assert blocking(small, "the stream is idle as far as the component has seen") == 1
            before = lib.xccl_rocm_direct_launch_count()
            evs = []
            for rep in range(48):
                st, e = rocm.xccl_mem_component_reduce_multi_nb(c1, c2, cr, 1, chain.size, chain.stride, Dt.INT32, Op.SUM,
                                                                MemType.ROCM, None)
                assert st == Status.OK and e is not None
                evs.append(e)
            assert lib.xccl_rocm_direct_launch_count() - before == 48
            t0 = time.time()
            while rocm.xccl_mc_event_query(evs[-1]) == Status.INPROGRESS:
                assert time.time() - t0 < 20.0
            for e in evs:
                assert rocm.xccl_mc_event_query(e) == Status.OK
                assert rocm.xccl_mc_event_free(e) == Status.OK
            a = chain.host[chain.o1: chain.o1 + chain.vbytes].view(np.int32).astype(np.int64)
            b = chain.host[chain.o2: chain.o2 + chain.vbytes].view(np.int32).astype(np.int64)
            want = ((a + 48 * b) & 0xffffffff).astype(np.uint32).view(np.int32)
            assert chain.result().view(np.int32).tolist() == want.tolist()
        finally:
            chain.close()
        # 2000 in a row: kernel-argument slots and packets are reused many times over
        p1, p2, pr = small.ptrs()
        before = lib.xccl_rocm_direct_launch_count()
        for rep in range(2000):
            assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, n2, small.size, small.stride, dt, op,
                                                        MemType.ROCM) == Status.OK
        assert lib.xccl_rocm_direct_launch_count() - before == 2000
        assert_same(small.result(), small.expect(oracle, op)[0], dt, op, "after 2000 calls")
    finally:
        lib.xccl_rocm_set_direct_queue(1)
        lib.xccl_rocm_set_direct_tail(1)
        small.close()
        large.close()


def test_many_events_in_flight_any_wait_order(rocm, oracle):
    """One pooled event per launch, 48 launches enqueued before the first wait,
    waited for in reverse order, mixed small (completion word) and large
    (HIP event) launches; then the pool is whole again."""
    dt, op = Dt.INT32, Op.BXOR
    cases, evs = [], []
    try:
        for k in range(48):
            size = (1 << 19) + 5 if k % 6 == 5 else 100 + 17 * k
            c = Case(dt, size, 1 + k % 3)
            c.fill_random(oracle, 50 + k)
            c.upload()
            cases.append(c)
        for c in cases:
            p1, p2, pr = c.ptrs()
            st, ev = rocm.xccl_mem_component_reduce_multi_nb(p1, p2, pr, c.n2, c.size, c.stride, dt, op, MemType.ROCM)
            assert st == Status.OK and ev
            evs.append(ev)
        for c, ev in reversed(list(zip(cases, evs))):
            assert rocm.xccl_mc_event_wait(ev) == Status.OK
            assert rocm.xccl_mc_event_query(ev) == Status.OK
            want, _ = c.expect(oracle, op)
            assert_same(c.result(), want, dt, op, "size %d" % c.size)
            assert rocm.xccl_mc_event_free(ev) == Status.OK
        s = rocm.Stream(hip.stream_create())
        got = []
        while True:
            st, ev = rocm.xccl_mc_event_record(s)
            if st != Status.OK:
                break
            got.append(ev)
        assert len(got) == 64
        for ev in got:
            rocm.xccl_mc_event_free(ev)
        hip.stream_destroy(s.hip_stream)
    finally:
        for c in cases:
            c.close()


def test_blocking_calls_from_several_threads(rocm, oracle):
    """test/test_mt.c runs 4 threads of collectives; the component's pools and
    lazy initialisation must hold up: 8 threads x 300 blocking reductions on
    private buffers, every result checked.  Eight threads share the four
    thread slots in pairs, so each of the component's own dispatch queues has
    two producers at once."""
    import threading
    dt, op, size = Dt.INT32, Op.SUM, 4096
    cases = []
    for t in range(8):
        c = Case(dt, size + t, 3)
        c.fill_random(oracle, 70 + t)
        c.upload()
        cases.append(c)
    errors = []

    def worker(c):
        try:
            p1, p2, pr = c.ptrs()
            want, _ = c.expect(oracle, op)
            for rep in range(300):
                st = rocm.xccl_mem_component_reduce_multi(p1, p2, pr, 3, c.size, c.stride, dt, op, MemType.ROCM)
                if st != Status.OK:
                    errors.append(st)
                    return
                if rep % 60 == 0:
                    assert_same(c.result(), want, dt, op, "thread size %d rep %d" % (c.size, rep))
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(c,)) for c in cases]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for c in cases:
        c.close()
    assert not errors, errors


def test_blocking_entry_through_graph_path(rocm, oracle):
    """XCCL_MC_ROCM_GRAPH_MAX_BYTES routes small blocking reductions through the
    cached single-node graph (read by open()); results must not change, and
    larger vectors keep the plain launch."""
    import os
    vt = rocm.component().super
    os.environ["XCCL_MC_ROCM_GRAPH_MAX_BYTES"] = "8192"
    try:
        assert vt.open() == Status.OK
        for rep in range(3):
            for dt, op, size, n2 in ((Dt.FLOAT32, Op.SUM, 2048, 3), (Dt.FLOAT32, Op.SUM, 2049, 3),
                                     (Dt.INT16, Op.MAX, 4096, 7), (Dt.FLOAT64, Op.PROD, 1000, 1),
                                     (Dt.UINT8, Op.BOR, 8192, 2), (Dt.INT32, Op.SUM, 1, 15)):
                c = Case(dt, size, n2)
                try:
                    c.fill_random(oracle, 90 + rep, op)
                    c.upload()
                    p1, p2, pr = c.ptrs()
                    assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, n2, size, c.stride, dt, op,
                                                                MemType.ROCM) == Status.OK
                    want, _ = c.expect(oracle, op)
                    assert_same(c.result(), want, dt, op, "graph-routed %s %s %d" % (Dt(dt).name, Op(op).name, size))
                finally:
                    c.close()
    finally:
        del os.environ["XCCL_MC_ROCM_GRAPH_MAX_BYTES"]
        assert vt.open() == Status.OK
        rocm.component_lib().xccl_rocm_graph_cache_destroy()


def test_stream_ordered_entries_under_stream_capture(rocm, oracle):
    """A caller records a whole k-nomial step sequence -- three dependent
    reduce_multi_nb launches on its own stream, no events -- into a hipGraph
    and replays it.  Every replay, with eager work and synchronisation in
    between, must reproduce the eager result (the entries enqueue kernels only:
    no memset nodes, no allocation)."""
    dt, op, size, n2 = Dt.FLOAT32, Op.SUM, 50000, 3
    c = Case(dt, size, n2)
    s = rocm.Stream(hip.stream_create())
    try:
        c.fill_random(oracle, 33)
        c.upload()
        p1, p2, pr = c.ptrs()

        def enqueue():
            for first in (p1, pr, pr):     # round 1 reads sbuf1, later rounds run in place on rbuf
                st, ev = rocm.xccl_mem_component_reduce_multi_nb(first, p2, pr, n2, size, c.stride, dt, op,
                                                                 MemType.ROCM, s, want_event=False)
                assert st == Status.OK and not ev

        enqueue()
        hip.stream_synchronize(s.hip_stream)
        eager = c.result().copy()
        img = c.host.copy()
        b = img.ctypes.data
        for first in (c.o1, c.orr, c.orr):
            oracle.reduce_multi_ptr(b + first, b + c.o2, b + c.orr, n2, size, c.stride, dt, op)
        assert_same(eager, img[c.orr: c.orr + c.vbytes], dt, op, "eager chain")

        hip.stream_begin_capture(s.hip_stream)
        enqueue()
        graph = hip.stream_end_capture(s.hip_stream)
        gexec = hip.graph_instantiate(graph)
        for rep in range(4):
            hip.memset(pr, 0x3C, c.vbytes)
            hip.graph_launch(gexec, s.hip_stream)
            hip.stream_synchronize(s.hip_stream)
            assert_same(c.result(), eager, dt, op, "graph replay %d" % rep)
            # eager work of the component between replays
            assert rocm.xccl_mem_component_reduce(p1, p2, pr, size, dt, op, MemType.ROCM) == Status.OK
        hip.graph_destroy(graph, gexec)
    finally:
        c.close()
        hip.stream_destroy(s.hip_stream)


def test_first_use_of_a_device_inside_a_capture_is_refused():
    """The component creates its per-device stream, events and counters on the
    first call on a device, which allocates and synchronises; inside a stream
    capture that would invalidate the capture.  A fresh process whose first
    call arrives with a capturing stream gets XCCL_ERR_NO_RESOURCE and an
    intact capture; after one call outside a capture the same capture works."""
    import os
    import subprocess
    import sys
    code = (
        "import sys\n"
        "sys.path.insert(0, %r)\n"
        "import numpy as np\n"
        "from xccl_amd import hip, mc\n"
        "from xccl_amd.types import Dt, MemType, Op, Status\n"
        "hip.set_device(0)\n"
        "assert mc.xccl_mem_component_init() == Status.OK\n"
        "buf = hip.DeviceBuffer(3 * 4096)\n"
        "buf.upload(np.arange(2048, dtype=np.float32))\n"
        "s = mc.Stream(hip.stream_create())\n"
        "args = (buf.ptr, buf.ptr + 4096, buf.ptr + 8192, 1, 1024, 4096, Dt.FLOAT32, Op.SUM, MemType.ROCM, s)\n"
        "hip.stream_begin_capture(s.hip_stream)\n"
        "first, _ = mc.xccl_mem_component_reduce_multi_nb(*args, want_event=False)\n"
        "g = hip.stream_end_capture(s.hip_stream)\n"          # the capture itself must have survived
        "hip.graph_destroy(g)\n"
        "warm = mc.xccl_mem_component_reduce_multi(*args[:9])\n"
        "hip.stream_begin_capture(s.hip_stream)\n"
        "second, _ = mc.xccl_mem_component_reduce_multi_nb(*args, want_event=False)\n"
        "g = hip.stream_end_capture(s.hip_stream)\n"
        "ge = hip.graph_instantiate(g)\n"
        "hip.memset(buf.ptr + 8192, 0, 4096)\n"
        "hip.graph_launch(ge, s.hip_stream)\n"
        "hip.stream_synchronize(s.hip_stream)\n"
        "got = buf.download(np.float32, 1024, 8192)\n"
        "ok = bool((got == np.arange(1024, dtype=np.float32) + np.arange(1024, 2048, dtype=np.float32)).all())\n"
        "print('first', int(first), 'warm', int(warm), 'second', int(second), 'replay', ok)\n"
    ) % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "first %d warm 0 second 0 replay True" % int(Status.ERR_NO_RESOURCE) in out.stdout, out.stdout + out.stderr
    assert "inside a stream capture" in out.stderr


def test_component_works_again_after_close():
    """close() releases a device's streams, events, dispatch queues and the
    code loaded for them -- after everything queued there has completed, also
    launches whose event nobody waited for; the next call sets everything up
    again.  A fresh process: small and large reductions on the own queue,
    four unwaited ones, close (through the dispatcher's free_cache), the same
    reductions once more."""
    import os
    import subprocess
    import sys
    code = (
        "import sys\n"
        "sys.path.insert(0, %r)\n"
        "import numpy as np\n"
        "from xccl_amd import hip, mc\n"
        "from xccl_amd.types import Dt, MemType, Op, Status\n"
        "hip.set_device(0)\n"
        "assert mc.xccl_mem_component_init() == Status.OK\n"
        "lib = mc.component_lib()\n"
        "n = 1 << 22\n"
        "buf = hip.DeviceBuffer(3 * n * 4)\n"
        "buf.upload(np.arange(2 * n, dtype=np.float32))\n"
        "want = np.arange(n, dtype=np.float32) + np.arange(n, 2 * n, dtype=np.float32)\n"
        "def run(count):\n"
        "    hip.memset(buf.ptr + 2 * n * 4, 0, count * 4)\n"
        "    hip.device_synchronize()\n"
        "    before = lib.xccl_rocm_direct_launch_count()\n"
        "    st = mc.xccl_mem_component_reduce_multi(buf.ptr, buf.ptr + n * 4, buf.ptr + 2 * n * 4, 1, count, n * 4,\n"
        "                                            Dt.FLOAT32, Op.SUM, MemType.ROCM)\n"
        "    got = buf.download(np.float32, count, 2 * n * 4)\n"
        "    return int(st), int(lib.xccl_rocm_direct_launch_count() - before), bool((got == want[:count]).all())\n"
        "a = [run(1000), run(1000), run(n)]\n"
        "# launches nobody waits for, on the own queue and on the stream, are still in flight when the component closes\n"
        "for count in (1000, n // 2, 1000, n):\n"
        "    st, ev = mc.xccl_mem_component_reduce_multi_nb(buf.ptr, buf.ptr + n * 4, buf.ptr + 2 * n * 4, 1, count, n * 4,\n"
        "                                                   Dt.FLOAT32, Op.SUM, MemType.ROCM, None)\n"
        "    assert st == Status.OK and ev\n"
        "mc.xccl_mem_component_free_cache()\n"
        "got = buf.download(np.float32, n, 2 * n * 4)\n"
        "assert (got == want).all(), 'close() did not wait for the launches in flight'\n"
        "b = [run(1000), run(1000), run(n)]\n"
        "print('before', a, 'after', b)\n"
    ) % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    expect = "[(0, 1, True), (0, 1, True), (0, 1, True)]"
    assert "before %s after %s" % (expect, expect) in out.stdout, out.stdout + out.stderr


def test_graph_launch_with_completion_word(rocm, oracle):
    """xccl_rocm_reduce_multi_graph_flagged: the one-node graph launch that
    carries the kernel-written completion word (its sequence number is a kernel
    argument, so every call patches the node) and reports the host time of its
    steps.  Same bits as the oracle on every call, the word written last."""
    lib = rocm.component_lib()
    stream = rocm.component_stream()
    host_word = hip.host_malloc(64)
    ctypes.memset(host_word, 0, 64)
    dev_word = hip.host_get_device_pointer(host_word)
    counters = hip.malloc((1 + 64) * 128)
    hip.memset(counters, 0, (1 + 64) * 128)
    hip.device_synchronize()
    word = ctypes.cast(host_word, ctypes.POINTER(ctypes.c_uint32))
    cases = []
    try:
        seq = 0
        for k, (dt, op, size, n2) in enumerate(((Dt.FLOAT32, Op.SUM, 4099, 3), (Dt.INT16, Op.MIN, 100000, 7),
                                                (Dt.FLOAT32, Op.SUM, 4099, 3), (Dt.UINT8, Op.LAND, 77, 1))):
            c = Case(dt, size, n2)
            c.fill_random(oracle, 90 + k, op)
            c.upload()
            cases.append(c)
            p1, p2, pr = c.ptrs()
            want, _ = c.expect(oracle, op)
            for rep in range(2):
                hip.memset(pr, 0xEE, c.vbytes)
                hip.device_synchronize()
                seq += 1
                flagged = ctypes.c_int(0)
                parts = (ctypes.c_uint64 * 4)()
                st = lib.xccl_rocm_reduce_multi_graph_flagged(p1, p2, pr, n2, size, c.stride, int(dt), int(op), stream,
                                                              counters, dev_word, seq, ctypes.byref(flagged), parts)
                assert st == Status.OK and flagged.value == 1
                t0 = time.time()
                while word[0] != seq:
                    assert time.time() - t0 < 20.0, "completion word never written"
                assert_same(c.result(), want, dt, op, "graph + completion word, %s %s rep %d" % (dt.name, op.name, rep))
                assert parts[3] > 0        # hipGraphLaunch took measurable host time
        # without a word it is the plain graph launch
        c = cases[0]
        p1, p2, pr = c.ptrs()
        assert lib.xccl_rocm_reduce_multi_graph_flagged(p1, p2, pr, c.n2, c.size, c.stride, int(Dt.FLOAT32), int(Op.SUM),
                                                        stream, None, None, 0, None, None) == Status.OK
        hip.stream_synchronize(stream)
    finally:
        hip.stream_synchronize(stream)
        for c in cases:
            c.close()
        lib.xccl_rocm_graph_cache_destroy()
        hip.free(counters)
        hip.host_free(host_word)
