"""GPU parity: the component, called through the dispatcher's C ABI, against the
CPU oracle on the same seeded bytes.  Bit-exact for every integer, logical,
bitwise, MIN and MAX case; floating-point SUM/PROD are folded in the same order
with one IEEE rounding per step, so they are compared bit-exact too (0 ULP),
except that a NaN result may carry any NaN encoding."""
import itertools

import numpy as np
import pytest

from gpu_util import NP, Case, assert_same, run_and_check
from xccl_amd.types import Dt, MemType, Op, Status, dt_size, supported_pairs, INT_DTYPES, FP_DTYPES, INT_OPS, FP_OPS

pytestmark = pytest.mark.gpu

ALL_PAIRS = supported_pairs()


def _id(p):
    return "%s-%s" % (Dt(p[0]).name, Op(p[1]).name)


@pytest.mark.parametrize("pair", ALL_PAIRS, ids=_id)
def test_every_dtype_op_small(rocm, oracle, pair):
    """Every supported (dtype, op): even and odd source counts (the walk
    through the sources alternates between two load registers), 2 to 17
    sources, sizes around the 16-byte vector and the 64-vector tile of a
    one-wave workgroup."""
    dt, op = pair
    for n2, size in ((1, 1), (1, 1000), (2, 37), (3, 4099), (4, 513), (7, 2048 + 5), (8, 700), (15, 1031),
                     (16, 129)):
        run_and_check(rocm, oracle, dt, op, size, n2, seed=int(dt) * 100 + int(op))


@pytest.mark.parametrize("dt", [Dt.INT8, Dt.UINT16, Dt.FLOAT16, Dt.INT32, Dt.FLOAT32, Dt.INT64, Dt.FLOAT64], ids=lambda d: Dt(d).name)
def test_misaligned_pointers_and_odd_strides(rocm, oracle, dt):
    """sbuf1, sbuf2 and rbuf at independent element offsets, strides that are
    not multiples of 16 bytes (scatter-reduce segments are arbitrary,
    allreduce_sra.c:281-284), and a stride that is not a multiple of the
    element size (host semantics: stride is bytes)."""
    es = dt_size(dt)
    op = Op.SUM
    size = 3001
    for off1, off2, offr in ((0, 0, 0), (es, 0, 0), (0, es, 0), (0, 0, es), (es, 2 * es, 3 * es), (8, 8, 8),
                             (es, es, es)):
        for n2 in (1, 3, 7, 6):
            for pad in (0, es, 4 + (es if es < 4 else 0), 24):
                run_and_check(rocm, oracle, dt, op, size, n2, off1=off1, off2=off2, offr=offr,
                              stride=size * es + pad, seed=3)
    # byte-granular placement of everything: pointers not even element-aligned
    if es > 1:
        run_and_check(rocm, oracle, dt, op, 777, 3, off1=1, off2=3, offr=1, stride=777 * es + 1, seed=4)
        run_and_check(rocm, oracle, dt, Op.MAX, 777, 4, off1=1, off2=1, offr=1, stride=777 * es + 3, seed=4)


@pytest.mark.parametrize("pair", [(Dt.INT32, Op.SUM), (Dt.FLOAT32, Op.SUM), (Dt.FLOAT16, Op.MAX), (Dt.INT8, Op.BXOR),
                                  (Dt.FLOAT64, Op.PROD), (Dt.UINT16, Op.MIN)], ids=_id)
def test_in_place(rocm, oracle, pair):
    """rbuf == sbuf1 (allreduce_knomial.c:118-121 after the first round),
    rbuf == sbuf2{0} (reduce_linear.c:28-34: target == sbuf2).  rbuf equal to
    a LATER vector of sbuf2 is not a defined use: the reference accumulates in
    rbuf itself, so that vector is overwritten before it is read."""
    dt, op = pair
    for size in (5, 1024, 10007):
        for n2 in (1, 3, 5, 7):
            run_and_check(rocm, oracle, dt, op, size, n2, alias="s1", seed=5)
            run_and_check(rocm, oracle, dt, op, size, n2, alias=("s2", 0), seed=6)


def test_reference_known_answer_on_device(rocm):
    """test/test_mpi_cuda_allreduce.c:35-39 + test/test_mt.c:58: INT32 SUM,
    count 32, rank r contributes r + 1 + 12345 + i; expect P(P+1)/2 + P(i+12345).
    Rank 0's vector is sbuf1, the others arrive in scratch = sbuf2."""
    import json
    import os
    from xccl_amd import hip
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "int32_sum_count32.json")
    for case in json.load(open(golden))["cases"]:
        nranks, count = case["team_size"], case["count"]
        ranks = np.array(case["inputs"], dtype=np.int32)
        src = hip.DeviceBuffer(ranks.nbytes)
        dst = hip.DeviceBuffer(count * 4)
        src.upload(ranks)
        st = rocm.xccl_mem_component_reduce_multi(src.ptr, src.ptr + count * 4, dst.ptr, nranks - 1, count, count * 4,
                                                  Dt.INT32, Op.SUM, MemType.ROCM)
        assert st == Status.OK
        assert dst.download(np.int32, count).tolist() == case["expected"]
        src.close()
        dst.close()


def _fp_specials(dt):
    npdt = NP[int(dt)]
    fi = np.finfo(npdt)
    return np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, fi.max, -fi.max, fi.tiny, -fi.tiny,
                     fi.smallest_subnormal, -fi.smallest_subnormal, fi.smallest_subnormal * 3, fi.tiny / 2,
                     fi.eps, 1 + fi.eps, 0.5, 3.0, -2.5], dtype=npdt)


@pytest.mark.parametrize("dt", FP_DTYPES, ids=lambda d: Dt(d).name)
@pytest.mark.parametrize("op", FP_OPS, ids=lambda o: Op(o).name)
def test_float_special_values(rocm, oracle, dt, op):
    """All ordered triples of special values (signed zeros, infinities, NaN,
    subnormals, extremes) as (sbuf1, sbuf2{0}, sbuf2{1}): MIN/MAX must hand
    back the exact operand bits that `a > b ? a : b` picks with the new source
    first; SUM/PROD must keep subnormals (no flush) and round once per step."""
    sp = _fp_specials(dt)
    trip = np.array(list(itertools.product(range(sp.size), repeat=3)))
    size = trip.shape[0]
    c = Case(dt, size, 2)
    try:
        c.set_s1(sp[trip[:, 0]].copy())
        c.set_s2(0, sp[trip[:, 1]].copy())
        c.set_s2(1, sp[trip[:, 2]].copy())
        c.upload()
        p1, p2, pr = c.ptrs()
        assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, 2, size, c.stride, dt, op, MemType.ROCM) == Status.OK
        with np.errstate(all="ignore"):
            want, _ = c.expect(oracle, op)
        assert_same(c.result(), want, dt, op, "specials %s %s" % (Dt(dt).name, Op(op).name))
    finally:
        c.close()


@pytest.mark.parametrize("dt", INT_DTYPES, ids=lambda d: Dt(d).name)
def test_integer_edge_values(rocm, oracle, dt):
    """All pairs of extreme values per integer dtype, every operator: wrap-around
    of SUM/PROD, signed vs unsigned MIN/MAX, 0/1 results of the logical ops."""
    import cmodel
    bits, signed = cmodel.INT_INFO[int(dt)]
    vals = cmodel.edge_values(bits, signed)
    pairs = list(itertools.product(vals, vals))
    a = np.array([p[0] for p in pairs], dtype=NP[int(dt)])
    b = np.array([p[1] for p in pairs], dtype=NP[int(dt)])
    for op in INT_OPS:
        c = Case(dt, len(pairs), 1)
        try:
            c.set_s1(a)
            c.set_s2(0, b)
            c.upload()
            p1, p2, pr = c.ptrs()
            assert rocm.xccl_mem_component_reduce(p1, p2, pr, len(pairs), dt, op, MemType.ROCM) == Status.OK
            got = c.result().view(NP[int(dt)])
            want = [cmodel.int_op(int(op), x, y, bits, signed) for x, y in pairs]
            assert [int(v) for v in got] == want, (Dt(dt).name, Op(op).name)
        finally:
            c.close()


def test_count_zero_equals_count_one_and_size_zero(rocm, oracle):
    """mem_component.c:129-139: size == 0 touches nothing; count == 0 still
    folds sbuf2{0} once."""
    dt, op, size = Dt.INT32, Op.SUM, 1000
    c = Case(dt, size, 1)
    try:
        c.fill_random(oracle, 8)
        c.upload()
        p1, p2, pr = c.ptrs()
        before = c.image()
        assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, 3, 0, c.stride, dt, op, MemType.ROCM) == Status.OK
        assert np.array_equal(c.image(), before)
        assert rocm.xccl_mem_component_reduce_multi(p1, p2, pr, 0, size, c.stride, dt, op, MemType.ROCM) == Status.OK
        want, _ = c.expect(oracle, op, count=1)
        assert_same(c.result(), want, dt, op, "count=0")
        # the component entry itself (not only the dispatcher) accepts size 0
        vt = rocm.component().super
        assert vt.reduce_multi(p1, p2, pr, 3, 0, c.stride, int(dt), int(op)) == Status.OK
        assert vt.reduce(p1, p2, pr, 0, int(dt), int(op)) == Status.OK
    finally:
        c.close()


def test_unsupported_returns_status_and_writes_nothing(rocm):
    from xccl_amd import hip
    buf = hip.DeviceBuffer(4096)
    hip.memset(buf.ptr, 0x5A, 4096)
    ok = set(supported_pairs())
    for dt in Dt:
        for op in Op:
            if (dt, op) in ok:
                continue
            st = rocm.xccl_mem_component_reduce_multi(buf.ptr, buf.ptr + 1024, buf.ptr + 2048, 1, 16, 64, dt, op,
                                                      MemType.ROCM)
            assert st == Status.ERR_UNSUPPORTED, (dt, op, st)
            st = rocm.xccl_mem_component_reduce(buf.ptr, buf.ptr + 1024, buf.ptr + 2048, 16, dt, op, MemType.ROCM)
            assert st == Status.ERR_UNSUPPORTED, (dt, op, st)
    assert (buf.download(np.uint8, 4096) == 0x5A).all()
    buf.close()


@pytest.mark.parametrize("n2", [1, 2, 3, 4, 5, 6, 7, 8, 9, 14, 15, 16, 17, 31, 32, 100, 1000])
def test_source_counts(rocm, oracle, n2):
    """MAX_REQS = 32 caps the k-nomial radix at 17 (xccl_ucx_lib.h:65); cover
    every count up to there and far beyond (the any-count kernel), fp32 SUM,
    fp64 MAX and int16 PROD."""
    run_and_check(rocm, oracle, Dt.FLOAT32, Op.SUM, 6007, n2, seed=20 + n2)
    run_and_check(rocm, oracle, Dt.FLOAT64, Op.MAX, 1501, n2, seed=40 + n2)
    run_and_check(rocm, oracle, Dt.INT16, Op.PROD, 2503, n2, seed=60 + n2)


def test_grid_cap_and_ragged_tiles(rocm, oracle):
    """Sizes that leave a partial tile, with the grid capped low (1 and 64
    workgroups per compute unit) so that every workgroup loops over tiles, then
    residency caps at both ends of the range (3 workgroups per compute unit,
    which also exercises the clamp of the LDS request, and no cap)."""
    lib = rocm.component_lib()
    try:
        for bpc in (1, 64):
            lib.xccl_rocm_set_launch_shape(bpc, 0)
            for size in (256 * 4 * 2 * 256 + 13, 1 << 20, (1 << 20) + 4 * 255 + 3):
                run_and_check(rocm, oracle, Dt.FLOAT32, Op.SUM, size, 7, seed=9, check_untouched=False)
                run_and_check(rocm, oracle, Dt.INT8, Op.SUM, size, 2, seed=9, check_untouched=False)
        for resident in (1, 3, 32):
            lib.xccl_rocm_set_launch_shape(0, resident)
            for dt, op in ((Dt.FLOAT32, Op.SUM), (Dt.INT16, Op.MAX), (Dt.FLOAT64, Op.MIN)):
                run_and_check(rocm, oracle, dt, op, (1 << 20) + 77, 7, seed=10, check_untouched=False)
                run_and_check(rocm, oracle, dt, op, 1001, 4, off1=dt_size(dt), seed=10)
    finally:
        lib.xccl_rocm_set_launch_shape(0, 0)


def test_walk_and_burst_kernels_agree_with_the_oracle(rocm, oracle):
    """Small launches with four or more sources run the burst kernel (every
    load of a tile at once), larger ones the source-by-source walk.  Both are
    forced onto the same calls -- every supported (dtype, op), source counts
    around the burst length of 8 and its multiples, ragged sizes, in place --
    and must give the oracle's bytes."""
    lib = rocm.component_lib()
    pairs = supported_pairs()
    try:
        for max_grid in (0, 1 << 30):        # never / always (from four sources on)
            lib.xccl_rocm_set_burst_max_grid(max_grid)
            for i, (dt, op) in enumerate(pairs):
                n2 = (3, 7, 8, 9, 15, 16, 17, 24, 25)[i % 9]
                run_and_check(rocm, oracle, dt, op, 1000 + 37 * i, n2, seed=300 + i,
                              alias=[None, "s1", ("s2", 0)][i % 3])
            for n2 in (3, 4, 7, 8, 9, 16, 17, 33):
                run_and_check(rocm, oracle, Dt.FLOAT32, Op.SUM, 70001, n2, seed=77 + n2, off1=4, offr=8)
                run_and_check(rocm, oracle, Dt.FLOAT64, Op.MIN, 513, n2, seed=78 + n2)
            kernel = rocm.reduce_multi_plan(1 << 12, 1 << 13, 1 << 14, 7, 256, 1024, Dt.FLOAT32, Op.SUM)["kernel"]
            assert kernel.endswith("Lb1EEEvNS_10ReduceArgsE" if max_grid else "Lb0EEEvNS_10ReduceArgsE"), kernel
    finally:
        lib.xccl_rocm_set_burst_max_grid(-1)


def test_every_dtype_op_on_the_stream_path(rocm, oracle):
    """Blocking calls normally go out on the component's own dispatch queue,
    whose kernels are loaded from code objects embedded in the library; with
    that path switched off the same calls run the kernels of the HIP module on
    a HIP stream.  Every supported (dtype, op), both kernel forms."""
    lib = rocm.component_lib()
    try:
        lib.xccl_rocm_set_direct_queue(0)
        before = lib.xccl_rocm_direct_launch_count()
        for i, (dt, op) in enumerate(supported_pairs()):
            run_and_check(rocm, oracle, dt, op, 2000 + 11 * i, (1, 2, 5, 9)[i % 4], seed=500 + i)
        assert lib.xccl_rocm_direct_launch_count() == before
        lib.xccl_rocm_set_direct_queue(1)       # (the calls above were blocking: nothing is left on the stream)
        for i, (dt, op) in enumerate(supported_pairs()):
            run_and_check(rocm, oracle, dt, op, 2000 + 11 * i, (1, 2, 5, 9)[i % 4], seed=500 + i)
        assert lib.xccl_rocm_direct_launch_count() - before == len(supported_pairs())
    finally:
        lib.xccl_rocm_set_direct_queue(1)


def test_randomised_shapes(rocm, oracle):
    """400 reproducible random calls: any supported (dtype, op), 1..20 vectors
    in sbuf2, sizes up to a few tiles, independent byte placement of the three
    buffers (element-aligned or not), strides padded by arbitrary byte counts,
    optionally in place on sbuf1 or sbuf2{0}; each compared with the oracle,
    bytes outside rbuf included."""
    rng = np.random.default_rng(20240607)
    pairs = supported_pairs()
    for it in range(400):
        dt, op = pairs[int(rng.integers(len(pairs)))]
        es = dt_size(dt)
        n2 = int(rng.integers(1, 21))
        size = int(rng.choice([1, 2, 3, 15, 16, 17, 63, 64, 65, 127, 129, 1000, 2047, 4097, int(rng.integers(1, 20000))]))
        unit = es if rng.random() < 0.8 else 1            # mostly element-aligned, sometimes byte-aligned
        off = [int(rng.integers(0, 64 // unit)) * unit for _ in range(3)]
        pad = int(rng.integers(0, 5)) * unit * int(rng.choice([0, 1, 3, 16]))
        alias = [None, None, "s1", ("s2", 0)][int(rng.integers(4))]
        run_and_check(rocm, oracle, dt, op, size, n2, seed=1000 + it, off1=off[0], off2=off[1], offr=off[2],
                      stride=size * es + pad, alias=alias)
