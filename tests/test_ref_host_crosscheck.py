"""A convenience cross-check, no pin: the oracle against the host branch of the
reference's own dispatcher (reference src/utils/mem_component.c:107-148 ->
src/utils/reduce.h:113-140), compiled from the reference tree by
tests/refdispatch/Makefile against stand-in UCX headers.  Because of those
stand-ins this build counts for nothing as a reference build; the oracle's pins
are in tests/test_oracle_pins.py and stand without it.  It covers the five
dtypes the reference implements; INT8, the unsigned types and FLOAT16 have no
reference implementation to compare with.  Skipped where the object is not
built."""
import ctypes
import os

import numpy as np
import pytest

import cmodel
from xccl_amd import mc
from xccl_amd.types import Dt, MemType, Op

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_SO = os.path.join(ROOT, "tests", "refdispatch", "_build", "libref_mc_unpatched.so")
NP = {1: np.int16, 2: np.int32, 3: np.int64, 11: np.float32, 12: np.float64}
INT_OPS = (Op.MAX, Op.MIN, Op.SUM, Op.PROD, Op.LAND, Op.LOR, Op.LXOR, Op.BAND, Op.BOR, Op.BXOR)
FP_OPS = (Op.MAX, Op.MIN, Op.SUM, Op.PROD)
HOST = int(MemType.HOST)


@pytest.fixture(scope="module")
def ref():
    if not os.path.isfile(REF_SO):
        pytest.skip("%s not built (make -C tests/refdispatch needs the reference tree)" % REF_SO)
    return mc.bind_dispatcher(REF_SO)


def _values(dt, n, rng):
    if dt in (Dt.FLOAT32, Dt.FLOAT64):
        npdt = NP[int(dt)]
        fi = np.finfo(npdt)
        special = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, fi.tiny, -fi.tiny, fi.smallest_subnormal,
                            fi.max, -fi.max, fi.eps, 1.0 + fi.eps], dtype=npdt)
        body = (rng.standard_normal(n) * 10.0 ** rng.integers(-30, 30, n)).astype(npdt)
        return np.concatenate([special, body])
    bits, signed = cmodel.INT_INFO[int(dt)]
    edge = np.array(cmodel.edge_values(bits, signed), dtype=NP[int(dt)])
    info = np.iinfo(NP[int(dt)])
    body = rng.integers(info.min, info.max, n, dtype=NP[int(dt)], endpoint=True)
    body[rng.random(n) < 0.3] = 0          # logical operators need zeros
    return np.concatenate([edge, body])


def _bits(a):
    return a.view(np.uint8).tobytes()


def _same(a, b, fp_arith):
    """Bit for bit; a NaN that an addition or multiplication PRODUCED may differ
    in sign between two compilations of the same C (x86 gives -NaN for inf-inf)."""
    if fp_arith:
        na, nb = np.isnan(a), np.isnan(b)
        return np.array_equal(na, nb) and _bits(a[~na]) == _bits(b[~nb])
    return _bits(a) == _bits(b)


@pytest.mark.parametrize("dt", [Dt.INT16, Dt.INT32, Dt.INT64, Dt.FLOAT32, Dt.FLOAT64])
def test_two_source_reduce_matches_the_reference_host_branch(ref, oracle, dt):
    rng = np.random.default_rng(100 + int(dt))
    v = _values(dt, 40, rng)
    a = np.repeat(v, v.size)
    b = np.tile(v, v.size)
    for op in (INT_OPS if int(dt) < 10 else FP_OPS):
        want = np.zeros_like(a)
        got = np.zeros_like(a)
        assert oracle.dt_reduce(a, b, want, a.size, dt, op) == 0
        st = ref.xccl_mem_component_reduce(a.ctypes.data, b.ctypes.data, got.ctypes.data, a.size, int(dt), int(op), HOST)
        assert st == 0
        assert _same(got, want, int(dt) >= 10 and op in (Op.SUM, Op.PROD)), (dt, op)


@pytest.mark.parametrize("dt", [Dt.INT16, Dt.INT32, Dt.INT64, Dt.FLOAT32, Dt.FLOAT64])
@pytest.mark.parametrize("count", [0, 1, 2, 7])
def test_reduce_multi_matches_the_reference_host_branch(ref, oracle, dt, count):
    """Fold order, count == 0 behaving as count == 1, stride in bytes with
    padding between the vectors, and the in-place form rbuf == sbuf1."""
    rng = np.random.default_rng(7 * int(dt) + count)
    size, es = 1237, np.dtype(NP[int(dt)]).itemsize
    stride = size * es + 3 * es
    nvec = max(count, 1)
    s1 = _values(dt, size, rng)[:size].copy()
    rng.shuffle(s1)
    s2 = np.zeros(nvec * stride // es, dtype=NP[int(dt)])
    for j in range(nvec):
        s2[j * stride // es: j * stride // es + size] = rng.permutation(_values(dt, size, rng))[:size]
    for op in (INT_OPS if int(dt) < 10 else FP_OPS):
        fp_arith = int(dt) >= 10 and op in (Op.SUM, Op.PROD)
        want = np.zeros(size, dtype=s1.dtype)
        got = np.zeros(size, dtype=s1.dtype)
        assert oracle.reduce_multi(s1, s2, want, count, size, stride, dt, op) == 0
        st = ref.xccl_mem_component_reduce_multi(s1.ctypes.data, s2.ctypes.data, got.ctypes.data, count, size, stride,
                                                 int(dt), int(op), HOST)
        assert st == 0
        assert _same(got, want, fp_arith), (dt, op, count)
        a1, a2 = s1.copy(), s1.copy()
        oracle.reduce_multi(a1, s2, a1, count, size, stride, dt, op)
        ref.xccl_mem_component_reduce_multi(a2.ctypes.data, s2.ctypes.data, a2.ctypes.data, count, size, stride, int(dt),
                                            int(op), HOST)
        assert _same(a2, a1, fp_arith), (dt, op, count, "in place")


def test_unsupported_cases_match_the_reference_host_branch(ref, oracle):
    """reduce.h:36-67,87-90,135-137: a dtype outside the five and a
    floating-point dtype with a bitwise operator return -1; an integer dtype
    with AND/OR/XOR/MAXLOC/MINLOC returns 0 and leaves the target alone;
    reduce_multi drops the inner status and is always XCCL_OK; size == 0 does
    nothing."""
    a = np.arange(16, dtype=np.int32)
    b = np.arange(16, dtype=np.int32) * 3
    for dt, op in ((Dt.INT8, Op.SUM), (Dt.UINT32, Op.SUM), (Dt.FLOAT16, Op.SUM), (Dt.FLOAT32, Op.BAND),
                   (Dt.FLOAT64, Op.LXOR), (Dt.INT128, Op.SUM), (Dt.INT32, Op.AND), (Dt.INT64, Op.MAXLOC),
                   (Dt.INT16, Op.XOR)):
        got = np.full(16, 0x5A5A5A5A, dtype=np.int32)
        want = got.copy()
        rc_ref = ref.xccl_mem_component_reduce(a.ctypes.data, b.ctypes.data, got.ctypes.data, 2, int(dt), int(op), HOST)
        rc_or = oracle.dt_reduce(a, b, want, 2, dt, op)
        if oracle.lib().oracle_dtype_in_reference(int(dt)):
            assert rc_ref == rc_or, (dt, op)
        else:
            assert rc_ref == -1          # the oracle implements these dtypes, the reference refuses them
        if rc_ref != 0 or op in (Op.AND, Op.MAXLOC, Op.XOR):
            assert got.tolist() == [0x5A5A5A5A] * 16
        if oracle.lib().oracle_dtype_in_reference(int(dt)):
            st = ref.xccl_mem_component_reduce_multi(a.ctypes.data, b.ctypes.data, got.ctypes.data, 1, 2, 8, int(dt),
                                                     int(op), HOST)
            assert st == 0 == oracle.reduce_multi(a, b, want, 1, 2, 8, dt, op)
            assert got.tolist() == want.tolist()
    got = np.full(4, 7, dtype=np.int32)
    assert ref.xccl_mem_component_reduce_multi(a.ctypes.data, b.ctypes.data, got.ctypes.data, 3, 0, 16, int(Dt.INT32),
                                               int(Op.SUM), HOST) == 0
    assert got.tolist() == [7] * 4
    assert ref.xccl_mem_component_reduce(a.ctypes.data, b.ctypes.data, got.ctypes.data, 4, int(Dt.INT32), int(Op.SUM),
                                         int(MemType.ROCM)) == -22       # no component loaded: mem_component.c:116-118
    p = ctypes.c_void_p()
    assert ref.xccl_mem_component_alloc(ctypes.byref(p), 64, HOST) == 0 and p.value
    assert ref.xccl_mem_component_free(p, HOST) == 0
