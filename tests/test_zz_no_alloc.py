"""xccl_rocm_reduce_multi_flagged_static -- the entry for callers that must not
allocate (its arrival counters live in a static device array inside the
library) -- against xccl_rocm_reduce_multi_flagged, whose counters the caller
brings: same bits, on two calls in a row, the second with a smaller input.
Both through the C ABI of xccl_rocm_mem_component.so."""
import ctypes
import time

import numpy as np
import pytest

from xccl_amd import hip
from xccl_amd.types import Dt, Op, Status, dt_size

from gpu_util import Case, assert_same

pytestmark = pytest.mark.gpu

DONE_COUNT_BYTES = (1 + 64) * 128


def _wait_word(host_word, seq, stream, what):
    """Polls the completion word; a launch that never writes it fails the test instead of hanging it."""
    word = ctypes.cast(host_word, ctypes.POINTER(ctypes.c_uint32))
    t0 = time.time()
    while word[0] != seq:
        if time.time() - t0 > 20.0:
            hip.stream_synchronize(stream)
            raise AssertionError("%s: completion word reads %d, expected %d" % (what, word[0], seq))
    return True


def test_static_scratch_entry_matches_flagged_entry(rocm, oracle):
    lib = rocm.component_lib()
    stream = rocm.component_stream()
    host_word = hip.host_malloc(64)
    ctypes.memset(host_word, 0, 64)
    dev_word = hip.host_get_device_pointer(host_word)
    counters = hip.malloc(DONE_COUNT_BYTES)
    hip.memset(counters, 0, DONE_COUNT_BYTES)
    hip.device_synchronize()
    seq = 0
    cases = []
    try:
        # second call smaller than the first; then a few more shapes (ragged tiles, one workgroup, 8192 workgroups)
        for k, (dt, op, size, n2) in enumerate(((Dt.FLOAT32, Op.SUM, 1 << 20, 7), (Dt.FLOAT32, Op.SUM, 100003, 7),
                                                (Dt.INT16, Op.MAX, 777, 2), (Dt.UINT8, Op.LXOR, 5, 1),
                                                (Dt.FLOAT64, Op.MIN, 1 << 20, 3), (Dt.INT32, Op.BXOR, 2 * 1024 * 1024, 1))):
            c = Case(dt, size, n2, off2=dt_size(dt) * (k % 2))
            c.fill_random(oracle, 70 + k, op)
            c.upload()
            cases.append(c)
            p1, p2, pr = c.ptrs()
            want, _ = c.expect(oracle, op)

            # the existing entry: counters from the caller
            hip.memset(pr, 0xEE, c.vbytes)
            hip.device_synchronize()
            flagged = ctypes.c_int(0)
            seq += 1
            st = lib.xccl_rocm_reduce_multi_flagged(p1, p2, pr, n2, size, c.stride, int(dt), int(op), stream, counters,
                                                    dev_word, seq, ctypes.byref(flagged))
            assert st == Status.OK
            if flagged.value:
                _wait_word(host_word, seq, stream, "flagged %s" % dt.name)
            else:
                hip.stream_synchronize(stream)
            ref = c.result().copy()
            assert_same(ref, want, dt, op, "flagged entry vs oracle, %s %s size %d" % (dt.name, op.name, size))

            # the entry that allocates nothing: twice in a row on the same arguments, counters left over from the
            # first launch must not disturb the second
            for rep in range(2):
                hip.memset(pr, 0x11 * (rep + 1), c.vbytes)
                hip.device_synchronize()
                seq += 1
                st = lib.xccl_rocm_reduce_multi_flagged_static(p1, p2, pr, n2, size, c.stride, int(dt), int(op), stream,
                                                               dev_word, seq)
                assert st == Status.OK
                _wait_word(host_word, seq, stream, "static %s rep %d" % (dt.name, rep))
                got = c.result()
                assert got.tobytes() == ref.tobytes(), "static entry differs from flagged entry: %s %s size %d rep %d" % (
                    dt.name, op.name, size, rep)
    finally:
        hip.stream_synchronize(stream)
        for c in cases:
            c.close()
        hip.free(counters)
        hip.host_free(host_word)


def test_static_scratch_entry_limits(rocm):
    """More than 8192 workgroups (8 MiB per vector) is refused before anything is enqueued; so is a call
    without a completion word; an unsupported pair is refused; a zero size reduces nothing and still writes the word."""
    lib = rocm.component_lib()
    stream = rocm.component_stream()
    host_word = hip.host_malloc(64)
    ctypes.memset(host_word, 0, 64)
    dev_word = hip.host_get_device_pointer(host_word)
    n = 3 * 1024 * 1024                     # 12 MiB of fp32 per vector
    buf = hip.malloc(3 * n * 4)
    try:
        args = (buf, buf + n * 4, buf + 2 * n * 4, 1, n, n * 4, int(Dt.FLOAT32), int(Op.SUM), stream)
        assert lib.xccl_rocm_reduce_multi_flagged_static(*args, dev_word, 1) == Status.ERR_INVALID_PARAM
        assert lib.xccl_rocm_reduce_multi_flagged_static(*args, None, 1) == Status.ERR_INVALID_PARAM
        hip.stream_synchronize(stream)
        assert ctypes.cast(host_word, ctypes.POINTER(ctypes.c_uint32))[0] == 0
        small = (buf, buf + n * 4, buf + 2 * n * 4, 1, 0, n * 4, int(Dt.FLOAT32), int(Op.SUM), stream)
        # size 0: nothing to reduce, but a caller polling the word must not wait in vain -- it is written, in stream order
        hip.memset(buf + 2 * n * 4, 0x5A, 64)
        assert lib.xccl_rocm_reduce_multi_flagged_static(*small, dev_word, 2) == Status.OK
        word = ctypes.cast(host_word, ctypes.POINTER(ctypes.c_uint32))
        t0 = time.time()
        while word[0] != 2:
            assert time.time() - t0 < 20.0, "size == 0: the completion word was never written"
        hip.stream_synchronize(stream)
        probe = np.empty(64, dtype=np.uint8)
        hip.memcpy_dtoh(probe, buf + 2 * n * 4)
        assert (probe == 0x5A).all()                                                                # and nothing else is
        bad = (buf, buf + n * 4, buf + 2 * n * 4, 1, 16, n * 4, int(Dt.FLOAT32), int(Op.BAND), stream)
        assert lib.xccl_rocm_reduce_multi_flagged_static(*bad, dev_word, 3) == Status.ERR_UNSUPPORTED
        bad0 = (buf, buf + n * 4, buf + 2 * n * 4, 1, 0, n * 4, int(Dt.FLOAT32), int(Op.BAND), stream)
        assert lib.xccl_rocm_reduce_multi_flagged_static(*bad0, dev_word, 4) == Status.ERR_UNSUPPORTED
        hip.stream_synchronize(stream)
        assert word[0] == 2
    finally:
        hip.free(buf)
        hip.host_free(host_word)
