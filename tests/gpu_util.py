"""Shared helpers of the GPU parity tests: lay sources out in one device
allocation, run the component through the dispatcher's C ABI, run the CPU
oracle on the same bytes, compare."""
import os

import numpy as np

from xccl_amd import hip
from xccl_amd.types import Dt, MemType, Op, Status, dt_size

NP = {0: np.int8, 1: np.int16, 2: np.int32, 3: np.int64, 5: np.uint8, 6: np.uint16, 7: np.uint32, 8: np.uint64,
      10: np.float16, 11: np.float32, 12: np.float64}
UINT = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}
LOGICAL = (Op.LAND, Op.LOR, Op.LXOR)
THREADS = max(1, min(16, os.cpu_count() or 1))


def is_fp(dt):
    return int(dt) in (10, 11, 12)


def assert_same(got: np.ndarray, want: np.ndarray, dt, op, what=""):
    """Bit-exact, except that a floating-point SUM/PROD whose result is NaN may
    carry any NaN encoding (x86 and the GPU pick different payloads when an
    operation produces or propagates a NaN; the reference does not define one)."""
    es = dt_size(dt)
    g = got.view(UINT[es])
    w = want.view(UINT[es])
    if is_fp(dt) and op in (Op.SUM, Op.PROD):
        gn, wn = np.isnan(got.view(NP[int(dt)])), np.isnan(want.view(NP[int(dt)]))
        assert np.array_equal(gn, wn), "%s: NaN positions differ" % what
        g, w = g[~wn], w[~wn]
    if not np.array_equal(g, w):
        bad = np.flatnonzero(g != w)
        i = int(bad[0])
        raise AssertionError("%s: %d of %d elements differ; first at %d: got %#x want %#x" %
                             (what, bad.size, g.size, i, int(g[i]), int(w[i])))


class Case:
    """One reduce_multi call: sbuf1, `n2` strided vectors in sbuf2 and rbuf
    placed at chosen byte offsets inside one device allocation and one
    identical host image."""

    def __init__(self, dt, size, n2, *, stride=None, off1=0, off2=0, offr=0, gap=256, alias=None):
        self.dt, self.size, self.n2 = dt, size, n2
        es = dt_size(dt)
        self.vbytes = size * es
        self.stride = self.vbytes if stride is None else stride
        span2 = (max(n2, 1) - 1) * self.stride + self.vbytes
        r1 = 64 + gap                       # region starts, 64-aligned bases plus caller offsets
        r2 = r1 + _up(self.vbytes + 64, 64) + gap
        rr = r2 + _up(span2 + 64, 64) + gap
        total = rr + _up(self.vbytes + 64, 64) + gap
        self.o1, self.o2, self.orr = r1 + off1, r2 + off2, rr + offr
        if alias == "s1":
            self.orr = self.o1
        elif isinstance(alias, tuple):      # ("s2", j)
            self.orr = self.o2 + alias[1] * self.stride
        self.host = np.zeros(total, dtype=np.uint8)
        self.dev = hip.DeviceBuffer(total)

    def set_s1(self, v):
        self.host[self.o1: self.o1 + self.vbytes] = v.view(np.uint8)[: self.vbytes]

    def set_s2(self, j, v):
        o = self.o2 + j * self.stride
        self.host[o: o + self.vbytes] = v.view(np.uint8)[: self.vbytes]

    def fill_random(self, oracle, seed, op=Op.SUM):
        sparse = op in LOGICAL
        self.set_s1(oracle.fill(self.size, self.dt, seed, 1000, sparse, THREADS))
        for j in range(max(self.n2, 1)):
            self.set_s2(j, oracle.fill(self.size, self.dt, seed, j, sparse, THREADS))

    def upload(self):
        self.dev.upload(self.host)

    def ptrs(self):
        return self.dev.ptr + self.o1, self.dev.ptr + self.o2, self.dev.ptr + self.orr

    def expect(self, oracle, op, count=None):
        """Oracle result on a copy of the host image; returns (result bytes, whole image after)."""
        img = self.host.copy()
        n = self.n2 if count is None else count
        es = dt_size(self.dt)
        if any(v % es for v in (self.o1, self.o2, self.orr, self.stride)):
            # operands that are not element-aligned: give the CPU aligned copies
            # (the fold is element-wise, so placement cannot change the result)
            npdt = NP[int(self.dt)]
            s1 = np.frombuffer(img[self.o1: self.o1 + self.vbytes].tobytes(), dtype=npdt).copy()
            s2 = np.empty((max(n, 1), self.size), dtype=npdt)
            for j in range(max(n, 1)):
                o = self.o2 + j * self.stride
                s2[j] = np.frombuffer(img[o: o + self.vbytes].tobytes(), dtype=npdt)
            out = np.empty(self.size, dtype=npdt)
            oracle.reduce_multi(s1, s2, out, n, self.size, self.vbytes, self.dt, op, threads=THREADS)
            img[self.orr: self.orr + self.vbytes] = out.view(np.uint8)
        else:
            base = img.ctypes.data
            oracle.reduce_multi_ptr(base + self.o1, base + self.o2, base + self.orr, n, self.size, self.stride,
                                    self.dt, op, threads=THREADS)
        return img[self.orr: self.orr + self.vbytes].copy(), img

    def result(self):
        return self.dev.download(np.uint8, self.vbytes, self.orr)

    def image(self):
        return self.dev.download(np.uint8, self.host.size, 0)

    def close(self):
        self.dev.close()


def _up(x, a):
    return (x + a - 1) // a * a


def run_and_check(mc, oracle, dt, op, size, n2, seed=1, check_untouched=True, **kw):
    c = Case(dt, size, n2, **kw)
    try:
        c.fill_random(oracle, seed, op)
        c.upload()
        p1, p2, pr = c.ptrs()
        st = mc.xccl_mem_component_reduce_multi(p1, p2, pr, n2, size, c.stride, dt, op, MemType.ROCM)
        assert st == Status.OK, st
        want, img = c.expect(oracle, op)
        what = "%s %s size=%d n2=%d %s" % (Dt(dt).name, Op(op).name, size, n2, kw)
        if check_untouched:
            got_img = c.image()
            got = got_img[c.orr: c.orr + c.vbytes]
            assert_same(got, want, dt, op, what)
            # nothing outside rbuf may change
            mask = np.ones(img.size, dtype=bool)
            mask[c.orr: c.orr + c.vbytes] = False
            assert np.array_equal(got_img[mask], img[mask]), what + ": bytes outside rbuf changed"
        else:
            assert_same(c.result(), want, dt, op, what)
    finally:
        c.close()
