"""The benchmark configurations at full size, against the CPU oracle (run with
one thread per host core; bit-identical to the single-thread fold), plus
size-independent properties."""
import numpy as np
import pytest

from gpu_util import NP, THREADS, assert_same
from xccl_amd import hip
from xccl_amd.types import Dt, MemType, Op, Status, dt_size, INT_OPS

pytestmark = pytest.mark.gpu


def _full_case(rocm, oracle, dt, ops, nsrc, size, seed, sparse_ops=(Op.LAND, Op.LOR, Op.LXOR)):
    es = dt_size(dt)
    stride = size * es
    dev = hip.DeviceBuffer((nsrc + 1) * stride)
    dst = dev.ptr + nsrc * stride
    want = np.empty(size, dtype=NP[int(dt)])
    loaded = None
    try:
        for op in ops:
            sparse = op in sparse_ops
            if loaded != sparse:
                slab = oracle.slab(nsrc, size, dt, seed, sparse=sparse, threads=THREADS)
                dev.upload(slab)
                loaded = sparse
            print("case", Dt(dt).name, Op(op).name, "nsrc", nsrc, "size", size, flush=True)
            st = rocm.xccl_mem_component_reduce_multi(dev.ptr, dev.ptr + stride, dst, nsrc - 1, size, stride, dt, op,
                                                      MemType.ROCM)
            assert st == Status.OK
            got = dev.download(NP[int(dt)], size, nsrc * stride)
            oracle.reduce_multi(slab, slab, want, nsrc - 1, size, stride, dt, op, off2=stride, threads=THREADS)
            assert_same(got, want, dt, op, "%s %s full size" % (Dt(dt).name, Op(op).name))
    finally:
        dev.close()
    return slab, got


def test_config2_fp32_sum_8x256MiB(rocm, oracle):
    """Headline: 8 source vectors of 67,108,864 floats at stride 256 MiB, SUM,
    fold order src0..src7.  Expected 0 ULP against the same-order CPU fold;
    also within (N-1)*u*sum|x_i| of a float64 sum on a sample."""
    size, n = 67108864, 8
    slab, got = _full_case(rocm, oracle, Dt.FLOAT32, [Op.SUM], n, size, seed=2)
    idx = np.arange(0, size, 4099)
    exact = slab[:, idx].astype(np.float64).sum(axis=0)
    bound = (n - 1) * 2.0 ** -24 * np.abs(slab[:, idx].astype(np.float64)).sum(axis=0)
    assert (np.abs(got[idx].astype(np.float64) - exact) <= bound).all()


@pytest.mark.parametrize("dt", [Dt.INT8, Dt.INT16, Dt.INT32, Dt.INT64, Dt.UINT32, Dt.UINT64], ids=lambda d: Dt(d).name)
def test_config3_integer_sweep(rocm, oracle, dt):
    """4 sources x 16,777,216 elements, all ten operators, full-range values
    (logical operators: half the elements zero); memcmp-equal to the oracle."""
    _full_case(rocm, oracle, dt, list(INT_OPS), 4, 16777216, seed=3)


@pytest.mark.parametrize("dt", [Dt.UINT8, Dt.UINT16, Dt.FLOAT16, Dt.FLOAT32, Dt.FLOAT64], ids=lambda d: Dt(d).name)
def test_remaining_dtypes_every_operator_multi_megabyte(rocm, oracle, dt):
    """The element types the integer sweep leaves out, every operator each
    supports, 3 sources x (4 Mi + 37) elements: thousands of workgroups, a
    ragged last tile, and launches on either side of the completion-word
    switch depending on the element size."""
    ops = list(INT_OPS) if int(dt) < int(Dt.FLOAT16) else [Op.MAX, Op.MIN, Op.SUM, Op.PROD]
    _full_case(rocm, oracle, dt, ops, 3, (4 << 20) + 37, seed=6)


@pytest.mark.parametrize("dt", [Dt.FLOAT16, Dt.FLOAT64], ids=lambda d: Dt(d).name)
def test_config4_fp16_fp64_16_sources(rocm, oracle, dt):
    """16 sources (radix-16 step) x 33,554,432 elements, SUM/MAX/MIN.  MAX/MIN
    bit-exact; SUM compared bit-exact with the same-order CPU fold (tolerance
    stated for the record: <= 1 ULP), and within (N-1)*u*sum|x_i| of a
    higher-precision sum on a sample (u = 2^-11 for binary16, 2^-53 for
    binary64)."""
    size, n = 33554432, 16
    slab, got = _full_case(rocm, oracle, dt, [Op.MAX, Op.MIN, Op.SUM], n, size, seed=4)
    idx = np.arange(0, size, 8191)
    hi = np.longdouble if dt == Dt.FLOAT64 else np.float64
    exact = slab[:, idx].astype(hi).sum(axis=0)
    u = 2.0 ** -53 if dt == Dt.FLOAT64 else 2.0 ** -11
    bound = (n - 1) * u * np.abs(slab[:, idx].astype(hi)).sum(axis=0)
    assert (np.abs(got[idx].astype(hi) - exact) <= bound).all()


def test_config1_two_source_fp32(rocm, oracle):
    """dst = a + b, FLOAT32 SUM, 1,048,576 elements, seed 0, contiguous: the
    reference's CPU-runnable case, through `reduce`."""
    size = 1048576
    a = oracle.fill(size, Dt.FLOAT32, 0, 0)
    b = oracle.fill(size, Dt.FLOAT32, 0, 1)
    dev = hip.DeviceBuffer(3 * size * 4)
    dev.upload(a)
    dev.upload(b, size * 4)
    assert rocm.xccl_mem_component_reduce(dev.ptr, dev.ptr + size * 4, dev.ptr + 2 * size * 4, size, Dt.FLOAT32,
                                          Op.SUM, MemType.ROCM) == Status.OK
    got = dev.download(np.float32, size, 2 * size * 4)
    want = np.empty(size, dtype=np.float32)
    assert oracle.dt_reduce(a, b, want, size, Dt.FLOAT32, Op.SUM) == 0
    assert got.tobytes() == want.tobytes() == (a + b).tobytes()
    dev.close()


def test_properties_at_full_size(rocm, oracle):
    """Size-independent properties on the headline shape, no oracle needed:
    XOR of a vector with itself an even number of times is zero; MAX then MIN
    of identical vectors is the vector; SUM of v and 7 zero vectors is v."""
    size, n = 67108864, 8
    stride = size * 4
    dev = hip.DeviceBuffer((n + 1) * stride)
    dst = dev.ptr + n * stride
    for j in range(n):
        assert rocm.datagen_fill(dev.ptr + j * stride, size, Dt.UINT32, 77, 0) == Status.OK   # 8 equal vectors
    hip.device_synchronize()
    v = dev.download(np.uint32, size, 0)
    run = lambda dt, op: rocm.xccl_mem_component_reduce_multi(dev.ptr, dev.ptr + stride, dst, n - 1, size, stride, dt,
                                                              op, MemType.ROCM)
    assert run(Dt.UINT32, Op.BXOR) == Status.OK
    assert not dev.download(np.uint32, size, n * stride).any()
    for op in (Op.MAX, Op.MIN, Op.BAND, Op.BOR):
        assert run(Dt.UINT32, op) == Status.OK
        assert np.array_equal(dev.download(np.uint32, size, n * stride), v)
    assert run(Dt.UINT32, Op.SUM) == Status.OK
    assert np.array_equal(dev.download(np.uint32, size, n * stride), v * np.uint32(8))
    hip.memset(dev.ptr + stride, 0, (n - 1) * stride)
    assert run(Dt.FLOAT32, Op.SUM) == Status.OK        # v + 0 + ... + 0 (as floats: x + 0 == x unless x is -0/NaN)
    f = v.view(np.float32)
    g = dev.download(np.float32, size, n * stride)
    ok = ~np.isnan(f) & (v != 0x80000000)
    assert np.array_equal(g.view(np.uint32)[ok], v[ok])
    dev.close()


def test_vectors_beyond_4GiB(rocm, oracle):
    """Vectors larger than 2^32 bytes (the device has 288 GB; the scatter-reduce
    path hands over whatever the user's buffer is): 64-bit indexing end to end.
    Three 5 GiB float vectors; windows at the start, across the 4 GiB line, and
    at the ragged end are compared with the oracle run on the same bytes."""
    size = 5 * (1 << 28) + 3                      # 1,342,177,283 floats = 5 GiB + 12 B
    stride = (size * 4 + 255) // 256 * 256
    free_b, _ = hip.mem_get_info()
    if free_b < 3 * stride + (1 << 30):
        pytest.skip("not enough free device memory")
    dev = hip.DeviceBuffer(3 * stride)
    try:
        for j in range(2):
            assert rocm.datagen_fill(dev.ptr + j * stride, size, Dt.FLOAT32, 9, j) == Status.OK
        hip.device_synchronize()
        assert rocm.xccl_mem_component_reduce_multi(dev.ptr, dev.ptr + stride, dev.ptr + 2 * stride, 1, size, stride,
                                                    Dt.FLOAT32, Op.SUM, MemType.ROCM) == Status.OK
        win = 1 << 18
        for lo in (0, (1 << 30) - win // 2, size - win):      # element 2^30 sits at byte 2^32
            a = dev.download(np.float32, win, lo * 4)
            b = dev.download(np.float32, win, stride + lo * 4)
            got = dev.download(np.float32, win, 2 * stride + lo * 4)
            want = np.empty(win, dtype=np.float32)
            assert oracle.dt_reduce(a, b, want, win, Dt.FLOAT32, Op.SUM) == 0
            assert got.tobytes() == want.tobytes(), "window at element %d" % lo
            assert np.count_nonzero(a) > win // 2 and np.count_nonzero(b) > win // 2
        # byte kernel with three sources, same footprint
        assert rocm.xccl_mem_component_reduce_multi(dev.ptr, dev.ptr + stride, dev.ptr + 2 * stride, 1, size * 4, stride,
                                                    Dt.UINT8, Op.BXOR, MemType.ROCM) == Status.OK
        for lo in ((1 << 32) - 4096, size * 4 - 8192):
            a = dev.download(np.uint8, 8192, lo)
            b = dev.download(np.uint8, 8192, stride + lo)
            assert np.array_equal(dev.download(np.uint8, 8192, 2 * stride + lo), a ^ b)
    finally:
        dev.close()


def test_config5_small_message_grid(rocm, oracle):
    """The small-message sweep as a parity test: FLOAT32 SUM, 2, 4 and 8
    sources, 4 B .. 32 KiB per vector in powers of two, through the three ways
    a call can complete -- the blocking entry, reduce_multi_nb + event polling,
    and the single-node graph launch -- each bit-exact against the oracle's
    same-order fold."""
    maxb = 32768
    lib = rocm.component_lib()
    stream = rocm.component_stream()
    slab = oracle.slab(8, maxb // 4, Dt.FLOAT32, 5)
    dev = hip.DeviceBuffer(9 * maxb)
    dev.upload(slab)
    dst = dev.ptr + 8 * maxb
    want = np.empty(maxb // 4, dtype=np.float32)
    try:
        for nsrc in (2, 4, 8):
            for k in range(14):
                nbytes = 4 << k
                cnt = nbytes // 4
                oracle.reduce_multi(slab, slab, want, nsrc - 1, cnt, maxb, Dt.FLOAT32, Op.SUM, off2=maxb)
                for mode in ("sync", "event", "graph"):
                    hip.memset(dst, 0xEE, maxb)
                    hip.device_synchronize()
                    if mode == "sync":
                        st = rocm.xccl_mem_component_reduce_multi(dev.ptr, dev.ptr + maxb, dst, nsrc - 1, cnt, maxb,
                                                                  Dt.FLOAT32, Op.SUM, MemType.ROCM)
                        assert st == Status.OK
                    elif mode == "event":
                        st, ev = rocm.xccl_mem_component_reduce_multi_nb(dev.ptr, dev.ptr + maxb, dst, nsrc - 1, cnt, maxb,
                                                                         Dt.FLOAT32, Op.SUM, MemType.ROCM)
                        assert st == Status.OK and ev
                        while True:
                            q = rocm.xccl_mc_event_query(ev)
                            if q != Status.INPROGRESS:
                                break
                        assert q == Status.OK
                        assert rocm.xccl_mc_event_free(ev) == Status.OK
                    else:
                        st = lib.xccl_rocm_reduce_multi_graph(dev.ptr, dev.ptr + maxb, dst, nsrc - 1, cnt, maxb,
                                                              int(Dt.FLOAT32), int(Op.SUM), stream)
                        assert st == Status.OK
                        hip.stream_synchronize(stream)
                    got = dev.download(np.float32, maxb // 4, 8 * maxb)
                    assert got[:cnt].tobytes() == want[:cnt].tobytes(), (nsrc, nbytes, mode)
                    assert (got[cnt:].view(np.uint8) == 0xEE).all(), "bytes behind the result written: %s" % ((nsrc, nbytes, mode),)
    finally:
        dev.close()
        lib.xccl_rocm_graph_cache_destroy()
