"""Pins the CPU oracle (oracle/xccl_oracle.c) to things that do not come from
the oracle itself: the reference tests' known answer, C integer semantics
worked out on Python ints, numpy's IEEE arithmetic, and hand-derived truth
tables.  A dropped term, a swapped operand or a wrong operator column fails at
least one of these."""
import itertools
import json
import os

import numpy as np
import pytest

import cmodel
from xccl_amd.types import Dt, Op, dt_size

NP = {0: np.int8, 1: np.int16, 2: np.int32, 3: np.int64, 5: np.uint8, 6: np.uint16, 7: np.uint32, 8: np.uint64,
      10: np.float16, 11: np.float32, 12: np.float64}


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "int32_sum_count32.json")


def test_reference_known_answer_int32_sum(oracle):
    """tests/golden/int32_sum_count32.json = reference test/test_mt.c:58 (same
    inputs test/test_mpi_allreduce.c:18-21, test/test_mpi_cuda_allreduce.c:35-39):
    every rank contributes sbuf[i] = rank + 1 + 12345 + i, count 32, INT32 SUM;
    the result must be P(P+1)/2 + P(i + 12345).  One k-nomial step with radix P
    is a reduce_multi over P vectors."""
    cases = json.load(open(GOLDEN))["cases"]
    assert [c["team_size"] for c in cases] == list(range(2, 18))
    for c in cases:
        nranks, count = c["team_size"], c["count"]
        ranks = np.array(c["inputs"], dtype=np.int32)
        out = np.zeros(count, dtype=np.int32)
        rc = oracle.reduce_multi(ranks, ranks, out, nranks - 1, count, count * 4, Dt.INT32, Op.SUM, off2=count * 4)
        assert rc == 0
        assert out.tolist() == c["expected"]
        assert c["expected"] == [nranks * (nranks + 1) // 2 + nranks * (i + 12345) for i in range(count)]


@pytest.mark.parametrize("dt", sorted(cmodel.INT_INFO))
@pytest.mark.parametrize("op", cmodel.INT_OPS)
def test_integer_ops_against_c_semantics(oracle, dt, op):
    bits, signed = cmodel.INT_INFO[dt]
    rng = np.random.default_rng(1000 * dt + op)
    vals = cmodel.edge_values(bits, signed)
    lo = -(1 << (bits - 1)) if signed else 0
    hi = (1 << (bits - 1)) - 1 if signed else (1 << bits) - 1
    vals += [int(v) for v in rng.integers(lo, hi, size=24, dtype=np.int64 if bits < 64 or signed else np.uint64,
                                          endpoint=True)]
    pairs = list(itertools.product(vals, vals))
    a = np.array([p[0] for p in pairs], dtype=NP[dt])
    b = np.array([p[1] for p in pairs], dtype=NP[dt])
    out = np.zeros_like(a)
    assert oracle.dt_reduce(a, b, out, len(pairs), dt, op) == 0
    expect = [cmodel.int_op(op, x, y, bits, signed) for x, y in pairs]
    assert [int(v) for v in out] == expect


@pytest.mark.parametrize("dt", [Dt.FLOAT16, Dt.FLOAT32, Dt.FLOAT64])
def test_float_sum_prod_against_numpy(oracle, dt):
    """IEEE round-to-nearest-even, one rounding per operation: numpy's
    elementwise add/multiply on the same dtype is an independent
    implementation (for float16 numpy rounds a float32 result once)."""
    rng = np.random.default_rng(int(dt))
    n = 200000
    npdt = NP[int(dt)]
    info = np.finfo(npdt)
    bits = rng.integers(0, 1 << (8 * dt_size(dt)), size=2 * n, dtype=np.uint64).astype(
        {2: np.uint16, 4: np.uint32, 8: np.uint64}[dt_size(dt)])
    x = bits.view(npdt)
    x = x[np.isfinite(x)][: 2 * (n // 2 - 1000)]
    a, b = x[: x.size // 2].copy(), x[x.size // 2: 2 * (x.size // 2)].copy()
    # include subnormals and cancellation
    a[:100] = info.smallest_subnormal * np.arange(100).astype(npdt)
    b[:100] = info.tiny
    b[100:200] = -a[100:200] * npdt(1.0009765625)
    out = np.empty_like(a)
    with np.errstate(all="ignore"):
        assert oracle.dt_reduce(a, b, out, a.size, dt, Op.SUM) == 0
        exp = a + b
        assert np.array_equal(out.view(bits.dtype)[~np.isnan(exp)], exp.view(bits.dtype)[~np.isnan(exp)])
        assert np.array_equal(np.isnan(out), np.isnan(exp))
        assert oracle.dt_reduce(a, b, out, a.size, dt, Op.PROD) == 0
        exp = a * b
        assert np.array_equal(out.view(bits.dtype)[~np.isnan(exp)], exp.view(bits.dtype)[~np.isnan(exp)])
        assert np.array_equal(np.isnan(out), np.isnan(exp))


def _ternary_max(a, b):
    return a if a > b else b


def _ternary_min(a, b):
    return a if a < b else b


@pytest.mark.parametrize("dt", [Dt.FLOAT16, Dt.FLOAT32, Dt.FLOAT64])
def test_float_min_max_truth_table(oracle, dt):
    """`a > b ? a : b` / `a < b ? a : b` (reduce.h:14-15): on a tie or an
    unordered compare the SECOND operand comes back, so (+0,-0) -> -0,
    (-0,+0) -> +0, (NaN,x) -> x, (x,NaN) -> NaN.  Expected values come from
    Python floats (IEEE doubles; every test value is exact in binary16)."""
    npdt = NP[int(dt)]
    specials = [0.0, -0.0, 1.0, -1.0, float("inf"), float("-inf"), float("nan"), 0.5, -0.5, 2.0]
    pairs = list(itertools.product(specials, specials))
    a = np.array([p[0] for p in pairs], dtype=npdt)
    b = np.array([p[1] for p in pairs], dtype=npdt)
    out = np.empty_like(a)
    for op, fn in ((Op.MAX, _ternary_max), (Op.MIN, _ternary_min)):
        assert oracle.dt_reduce(a, b, out, len(pairs), dt, op) == 0
        for k, (x, y) in enumerate(pairs):
            e = fn(x, y)
            got = float(out[k])
            if e != e:
                assert got != got, (op, x, y, got)
            else:
                assert got == e and np.signbit(got) == np.signbit(e), (op, x, y, got)


def test_half_conversions_against_numpy(oracle):
    l = oracle.lib()
    halves = np.arange(65536, dtype=np.uint16)
    want = halves.view(np.float16).astype(np.float32)
    got = np.array([l.oracle_half_to_float(int(h)) for h in halves], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.array_equal(np.isnan(got), nan)

    rng = np.random.default_rng(7)
    f = rng.integers(0, 1 << 32, size=300000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    # every rounding boundary of binary16: halfway points between neighbours, and their float32 neighbours
    mids = []
    hs = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)
    for lo, hi in zip(hs[:-1], hs[1:]):
        m = np.float32((lo + hi) / 2)
        mids += [m, np.nextafter(m, np.float32(np.inf)), np.nextafter(m, np.float32(-np.inf))]
    edge = np.array(mids + [65504.0, 65519.996, 65520.0, 65536.0, 1e-8, 2.0 ** -25, 2.0 ** -24, 0.0], dtype=np.float32)
    f = np.concatenate([f, edge, -edge])
    f = f[~np.isnan(f)]
    with np.errstate(over="ignore"):
        want16 = f.astype(np.float16).view(np.uint16)
    got16 = np.array([l.oracle_float_to_half(float(v)) for v in f], dtype=np.uint16)
    assert np.array_equal(got16, want16)


def test_fold_order_is_new_source_first(oracle):
    """mem_component.c:133-139.  With MAX on signed zeros the result depends on
    which operand is first: acc = OP(s1, s2_0), then acc = OP(s2_j, acc).
    Expected values from the Python model of the fold, not from the oracle."""
    pz, nz = 0.0, -0.0
    cases = [
        (pz, [nz]), (nz, [pz]), (pz, [nz, pz]), (pz, [pz, nz]), (nz, [nz, pz, nz]),
        (nz, [pz, nz, nz]), (1.0, [float("nan"), 2.0]), (1.0, [2.0, float("nan")]),
        (float("nan"), [1.0, 0.5]), (pz, [nz, nz, nz, pz, nz, nz, nz]),
    ]
    for dt in (Dt.FLOAT16, Dt.FLOAT32, Dt.FLOAT64):
        for op, fn in ((Op.MAX, _ternary_max), (Op.MIN, _ternary_min)):
            for s1, s2 in cases:
                a = np.array([s1], dtype=NP[int(dt)])
                b = np.array(s2, dtype=NP[int(dt)])
                out = np.empty(1, dtype=NP[int(dt)])
                oracle.reduce_multi(a, b, out, len(s2), 1, dt_size(dt), dt, op)
                e = cmodel.fold(fn, s1, s2)
                g = float(out[0])
                assert (g != g and e != e) or (g == e and np.signbit(g) == np.signbit(e)), (dt, op, s1, s2, g, e)


@pytest.mark.parametrize("dt,op", [(Dt.INT32, Op.SUM), (Dt.FLOAT32, Op.SUM), (Dt.FLOAT64, Op.PROD),
                                   (Dt.FLOAT16, Op.SUM), (Dt.UINT8, Op.PROD), (Dt.INT64, Op.MIN),
                                   (Dt.FLOAT32, Op.MAX), (Dt.UINT16, Op.LXOR)])
def test_reduce_multi_is_chained_reduce(oracle, dt, op):
    """reduce_multi(N) == N-1 chained 2-source reduces with the operand order
    of mem_component.c:134-138; stride in bytes may exceed the vector."""
    size, nvec, pad = 1537, 6, 24
    stride = size * dt_size(dt) + pad
    s1 = oracle.fill(size, dt, 3, 100)
    raw = np.zeros(nvec * stride, dtype=np.uint8)
    vecs = []
    for j in range(nvec):
        v = oracle.fill(size, dt, 3, j, sparse=(op in (Op.LAND, Op.LOR, Op.LXOR)))
        raw[j * stride: j * stride + v.nbytes] = v.view(np.uint8)
        vecs.append(v)
    out = np.zeros(size, dtype=NP[int(dt)])
    assert oracle.reduce_multi(s1, raw, out, nvec, size, stride, dt, op) == 0
    acc = np.zeros_like(out)
    assert oracle.dt_reduce(s1, vecs[0], acc, size, dt, op) == 0
    for j in range(1, nvec):
        nxt = np.zeros_like(out)
        assert oracle.dt_reduce(vecs[j], acc, nxt, size, dt, op) == 0
        acc = nxt
    assert out.tobytes() == acc.tobytes()


def test_float_sum_left_fold_against_numpy(oracle):
    """((v0 + v1) + v2) + ... in source order, one rounding per step."""
    n, size = 8, 4096
    for dt in (Dt.FLOAT16, Dt.FLOAT32, Dt.FLOAT64):
        slab = oracle.slab(n, size, dt, 5)
        out = np.empty(size, dtype=NP[int(dt)])
        oracle.reduce_multi(slab, slab, out, n - 1, size, size * dt_size(dt), dt, Op.SUM, off2=size * dt_size(dt))
        acc = slab[0] + slab[1]
        for j in range(2, n):
            acc = slab[j] + acc
        assert out.tobytes() == acc.tobytes()


def test_size_zero_and_count_zero(oracle):
    a = np.array([1, 2, 3], dtype=np.int32)
    b = np.array([10, 20, 30, 100, 200, 300], dtype=np.int32)
    out = np.full(3, -7, dtype=np.int32)
    assert oracle.reduce_multi(a, b, out, 2, 0, 12, Dt.INT32, Op.SUM) == 0
    assert out.tolist() == [-7, -7, -7]  # mem_component.c:129-131
    out0 = np.zeros(3, dtype=np.int32)
    out1 = np.zeros(3, dtype=np.int32)
    oracle.reduce_multi(a, b, out0, 0, 3, 12, Dt.INT32, Op.SUM)  # first step still runs (:134)
    oracle.reduce_multi(a, b, out1, 1, 3, 12, Dt.INT32, Op.SUM)
    assert out0.tolist() == out1.tolist() == [11, 22, 33]


def test_unsupported_combinations(oracle):
    a = np.ones(4, dtype=np.int32)
    out = np.full(4, 9, dtype=np.int32)
    # dtypes outside the table: reduce.h:135-137
    for dt in (Dt.INT128, Dt.UINT128, Dt.LAST_PREDEFINED, Dt.UNSUPPORTED):
        assert oracle.dt_reduce(a, a, out, 1, dt, Op.SUM) == -1
    # floating point with a logical/bitwise operator: reduce.h:87-90
    f = np.ones(4, dtype=np.float32)
    fo = np.zeros(4, dtype=np.float32)
    for op in (Op.LAND, Op.LOR, Op.LXOR, Op.BAND, Op.BOR, Op.BXOR, Op.AND, Op.MAXLOC):
        assert oracle.dt_reduce(f, f, fo, 4, Dt.FLOAT32, op) == -1
    # integer dtype with an operator outside the switch: nothing written, returns 0 (reduce.h:36-67)
    for op in (Op.AND, Op.OR, Op.XOR, Op.MAXLOC, Op.MINLOC):
        assert oracle.dt_reduce(a, a, out, 4, Dt.INT32, op) == 0
        assert out.tolist() == [9, 9, 9, 9]
    assert [oracle.lib().oracle_dtype_in_reference(int(d)) for d in (Dt.INT8, Dt.INT16, Dt.INT32, Dt.INT64,
            Dt.UINT8, Dt.UINT32, Dt.FLOAT16, Dt.FLOAT32, Dt.FLOAT64)] == [0, 1, 1, 1, 0, 0, 0, 1, 1]


def test_in_place_aliasing(oracle):
    """Call sites alias rbuf with sbuf1 (allreduce_knomial.c:118-121) and
    target with sbuf2 (reduce_linear.c:28-34)."""
    size, n = 1000, 4
    dt, op = Dt.INT32, Op.SUM
    s1 = oracle.fill(size, dt, 9, 50)
    slab = oracle.slab(n, size, dt, 9)
    ref = np.empty(size, dtype=np.int32)
    oracle.reduce_multi(s1, slab, ref, n, size, size * 4, dt, op)
    inplace = s1.copy()
    oracle.reduce_multi(inplace, slab, inplace, n, size, size * 4, dt, op)
    assert np.array_equal(inplace, ref)
    slab2 = slab.copy()
    oracle.reduce_multi(s1, slab2, slab2, n, size, size * 4, dt, op)  # rbuf == sbuf2{0}
    assert np.array_equal(slab2[0], ref)
    t = slab[0].copy()
    oracle.dt_reduce(s1, t, t, size, dt, op)
    assert np.array_equal(t, s1 + slab[0])


def test_threaded_fold_is_bit_identical(oracle):
    size, n = 100003, 5
    for dt, op in ((Dt.FLOAT32, Op.SUM), (Dt.FLOAT16, Op.PROD), (Dt.INT8, Op.MAX), (Dt.FLOAT64, Op.SUM)):
        slab = oracle.slab(n + 1, size, dt, 11)
        es = dt_size(dt)
        a = np.empty(size, dtype=NP[int(dt)])
        b = np.empty(size, dtype=NP[int(dt)])
        oracle.reduce_multi(slab, slab, a, n, size, size * es, dt, op, off2=size * es, threads=1)
        oracle.reduce_multi(slab, slab, b, n, size, size * es, dt, op, off2=size * es, threads=7)
        assert a.tobytes() == b.tobytes()


def _splitmix64_np(z):
    z = (z + np.uint64(0x9E3779B97F4A7C15))
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def test_input_generator_recipe(oracle):
    """The synthetic-input recipe, recomputed with numpy uint64 arithmetic.
    splitmix64 itself is pinned by its published test vector (seed 1234567:
    first outputs 6457827717110365317, 3203168211198807973)."""
    s = 1234567
    o1 = oracle.lib().oracle_splitmix64(s)
    o2 = oracle.lib().oracle_splitmix64((s + 0x9E3779B97F4A7C15) & (2 ** 64 - 1))
    assert (o1, o2) == (6457827717110365317, 3203168211198807973)
    n, seed, vec = 5000, 3, 2
    with np.errstate(over="ignore"):
        base = np.uint64((seed * 0x9E3779B97F4A7C15 + (vec << 40)) & (2 ** 64 - 1))
        x = _splitmix64_np(base + np.arange(n, dtype=np.uint64))
        y = _splitmix64_np(x)
    f32 = (x >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -23) - np.float32(1.0)
    assert np.array_equal(oracle.fill(n, Dt.FLOAT32, seed, vec), f32)
    f16 = ((x >> np.uint64(53)).astype(np.float32) * np.float32(2.0 ** -11) - np.float32(0.5)).astype(np.float16)
    assert np.array_equal(oracle.fill(n, Dt.FLOAT16, seed, vec), f16)
    assert f32.min() >= -1.0 and f32.max() < 1.0 and f16.min() >= -0.5 and f16.max() < 0.5
    for dt, npdt in ((Dt.INT8, np.uint8), (Dt.UINT16, np.uint16), (Dt.INT32, np.uint32), (Dt.UINT64, np.uint64)):
        got = oracle.fill(n, dt, seed, vec).view(npdt)
        assert np.array_equal(got, x.astype(npdt))
        sparse = oracle.fill(n, dt, seed, vec, sparse=True).view(npdt)
        keep = (y >> np.uint64(63)) == 0
        assert np.array_equal(sparse, np.where(keep, x.astype(npdt), 0).astype(npdt))
        assert 0.4 < keep.mean() < 0.6
    d = oracle.fill(200000, Dt.FLOAT64, seed, vec)
    assert abs(d.mean()) < 0.01 and abs(d.std() - 1.0) < 0.01
    # threads do not change the stream
    assert np.array_equal(oracle.fill(200000, Dt.FLOAT64, seed, vec, threads=1), d)
